"""Mints the golden tables for the narrow-type conversions from the REFERENCE's own
number classes.  It loads oracle/_ref/libref_datatypes.so, which `make -C oracle`
compiles from the reference file
  mlir-tensorrt/executor/lib/Runtime/Backend/Common/DataTypes.cpp
where it lies (possible only where the reference tree is mounted), and writes

  lowp_from_f16_grid.npz   for every f16 bit pattern h: f32(h) (as the reference widens it), and
                           the reference's f8E4M3FN / bf16 / f16 narrowing of that f32 value
  lowp_f32_samples.npz     a stratified f32 sample (every f8/f16 rounding boundary +-1 ulp, the
                           ranges where the reference deviates from IEEE, seeded random bit
                           patterns) with the reference's f8 / f16 / bf16 results
  lowp_widen.npz           f8 -> f32 for all 256 codes, int4 constructor/sign-extension tables

Run from the repository root:  python tests/golden/make_lowp_golden.py
The outputs are data (inputs and expected outputs) and are committed; this script and
the library it loads are not needed to run the tests.
"""
import ctypes
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
import oracle.binding as ob  # noqa: E402


def main():
    R = ob.ref()
    if R is None:
        raise SystemExit("oracle/_ref/libref_datatypes.so is not built (needs the reference tree): make -C oracle")
    vp = ctypes.c_void_p

    def bulk(fn, x, dtype):
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.empty(x.size, dtype=dtype)
        fn(x.ctypes.data_as(vp), out.ctypes.data_as(vp), x.size)
        return out

    # 1. the f16 grid
    h = np.arange(65536, dtype=np.uint16)
    f32_of_h = np.array([R.ref_f16_to_f32(int(c)) for c in h], dtype=np.float32)
    np.savez_compressed(os.path.join(HERE, "lowp_from_f16_grid.npz"),
                        f32_bits=f32_of_h.view(np.uint32),
                        f8=bulk(R.ref_f32_to_f8e4m3fn_bulk, f32_of_h, np.uint8),
                        bf16=bulk(R.ref_f32_to_bf16_bulk, f32_of_h, np.uint16),
                        f16=bulk(R.ref_f32_to_f16_bulk, f32_of_h, np.uint16))

    # 2. stratified f32 sample
    parts = []
    f8_vals = np.array([R.ref_f8e4m3fn_to_f32(c) for c in range(0x7F)], dtype=np.float64)
    mids8 = ((f8_vals[:-1] + f8_vals[1:]) / 2).astype(np.float32)        # every f8 tie (exact in f32)
    f16_pos = f32_of_h[:0x7C00].astype(np.float64)
    mids16 = ((f16_pos[:-1] + f16_pos[1:]) / 2).astype(np.float32)[::7]   # every 7th f16 tie
    for m in (mids8, mids16, f8_vals.astype(np.float32)):
        parts += [m, np.nextafter(m, np.float32(np.inf)), np.nextafter(m, np.float32(-np.inf))]
    # where the reference's f8 deviates from IEEE: [240, 480] and the top of the subnormal range
    parts.append(np.linspace(240, 480, 4001, dtype=np.float32))
    parts.append(np.linspace(0.0135, 0.0160, 4001, dtype=np.float32))
    parts.append(np.linspace(5.9e-5, 6.2e-5, 2001, dtype=np.float32))     # top of the f16 subnormal range
    g = np.random.Generator(np.random.PCG64(20240601))
    parts.append(g.integers(0, 2**32, 20000, dtype=np.uint64).astype(np.uint32).view(np.float32))
    parts.append((g.standard_normal(8000) * 3).astype(np.float32))
    parts.append(np.float32([0.0, -0.0, np.inf, -np.inf, 448, 449, 464, 465, 1000, 1e-10, 0.005, 0.001,
                             65504, 65520, 65536, 3.4e38, 1e-40, 2.32356, 0.395264, 10.7, 200.0]))
    x = np.concatenate(parts)
    x = np.concatenate([x, -x])
    x = x[~np.isnan(x)]
    nan_bits = np.uint32([0x7FC00000, 0xFFC00000, 0x7F800001, 0x7FFFFFFF, 0xFFFFFFFF, 0x7FC12345])
    xb = np.concatenate([x.view(np.uint32), nan_bits])
    x = xb.view(np.float32)
    np.savez_compressed(os.path.join(HERE, "lowp_f32_samples.npz"),
                        x_bits=xb,
                        f8=bulk(R.ref_f32_to_f8e4m3fn_bulk, x, np.uint8),
                        f16=bulk(R.ref_f32_to_f16_bulk, x, np.uint16),
                        bf16=bulk(R.ref_f32_to_bf16_bulk, x, np.uint16))

    # 3. widening and int4 tables
    ints = np.arange(-40, 41, dtype=np.int32)
    fl = np.float32([-9.5, -8.99, -8.0, -7.5, -0.9, -0.0, 0.0, 0.9, 5.89699984, 6.99, 7.0, 7.01, 8.5, 100.0, -100.0])
    np.savez_compressed(os.path.join(HERE, "lowp_widen.npz"),
                        f8_to_f32_bits=np.array([R.ref_f8e4m3fn_to_f32(c) for c in range(256)], dtype=np.float32).view(np.uint32),
                        bf16_probe=np.uint16([0, 0x8000, 0x3F80, 0x7F80, 0xFF80, 0x7FC0, 0x0001, 0x7F7F]),
                        bf16_probe_f32_bits=np.array([R.ref_bf16_to_f32(int(c)) for c in
                                                      [0, 0x8000, 0x3F80, 0x7F80, 0xFF80, 0x7FC0, 0x0001, 0x7F7F]],
                                                     dtype=np.float32).view(np.uint32),
                        int4_in=ints,
                        int4_value=np.array([R.ref_int4_from_int(int(v)) for v in ints], dtype=np.int8),
                        int4_raw=np.array([R.ref_int4_raw_from_int(int(v)) for v in ints], dtype=np.uint8),
                        int4_from_raw=np.array([R.ref_int4_from_raw(c) for c in range(16)], dtype=np.int8),
                        fptosi_in=fl,
                        fptosi_i4=np.array([R.ref_fptosi_f32_i4(float(v)) for v in fl], dtype=np.int8))
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
