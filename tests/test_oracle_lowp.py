"""Pins oracle/lowp.hpp (CPU only):
  - refhost mode against golden tables minted from the compiled reference classes
    (tests/golden/make_lowp_golden.py) and, where oracle/_ref is built, against that
    library directly on fresh random inputs;
  - ieee mode against numpy float16 and torch bfloat16 / float8_e4m3fn casts;
  - both modes against the known answers the reference's own tests print.
The exhaustive 2^32 comparison lives in `make -C oracle pin`.
"""
import json
import math
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _load(name):
    return np.load(os.path.join(GOLD, name))


def test_refhost_matches_reference_on_f16_grid(orc):
    g = _load("lowp_from_f16_grid.npz")
    x = g["f32_bits"].view(np.float32)
    assert np.array_equal(orc.widen(np.arange(65536, dtype=np.uint16), orc.F16).view(np.uint32), g["f32_bits"])
    assert np.array_equal(orc.narrow(x, orc.F8E4M3FN, orc.REFHOST), g["f8"])
    assert np.array_equal(orc.narrow(x, orc.F16, orc.REFHOST), g["f16"])
    assert np.array_equal(orc.narrow(x, orc.BF16, orc.REFHOST), g["bf16"])


def test_refhost_matches_reference_on_stratified_f32(orc):
    g = _load("lowp_f32_samples.npz")
    x = g["x_bits"].view(np.float32)
    assert x.size > 100000
    assert np.array_equal(orc.narrow(x, orc.F8E4M3FN, orc.REFHOST), g["f8"])
    assert np.array_equal(orc.narrow(x, orc.F16, orc.REFHOST), g["f16"])
    assert np.array_equal(orc.narrow(x, orc.BF16, orc.REFHOST), g["bf16"])


def test_widen_and_int4_tables(orc):
    g = _load("lowp_widen.npz")
    assert np.array_equal(orc.widen(np.arange(256, dtype=np.uint8), orc.F8E4M3FN).view(np.uint32), g["f8_to_f32_bits"])
    assert np.array_equal(orc.widen(g["bf16_probe"], orc.BF16).view(np.uint32), g["bf16_probe_f32_bits"])
    L = orc.lib()
    assert [L.orc_int4_saturate(int(v)) for v in g["int4_in"]] == list(g["int4_value"])
    assert [L.orc_int4_saturate(int(v)) & 0xF for v in g["int4_in"]] == list(g["int4_raw"])
    assert [L.orc_int4_sign_extend(c) for c in range(16)] == list(g["int4_from_raw"])
    # _fptosi_f32_i4 = Int4(trunc(x)), saturating
    assert [L.orc_int4_saturate(int(math.trunc(float(v)))) for v in g["fptosi_in"]] == list(g["fptosi_i4"])


def test_reference_deviations_are_what_the_header_says(orc):
    """The three places where the host class leaves IEEE, as plain facts."""
    f8 = lambda v, m: int(orc.lib().orc_f32_to_f8e4m3fn(float(v), m))
    for v in (248.0, 256.0, 300.0, 447.0):                 # exponent-15 results collapse to 448
        assert f8(v, orc.REFHOST) == 0x7E
    assert [f8(v, orc.IEEE) for v in (248.0, 256.0, 300.0, 447.0)] == [0x78, 0x78, 0x79, 0x7E]
    assert f8(240.0, orc.REFHOST) == f8(240.0, orc.IEEE) == 0x77
    assert f8(0.0155, orc.REFHOST) == 0x00 and f8(0.0155, orc.IEEE) == 0x08   # lost carry into the least normal
    assert f8(17.0, orc.REFHOST) == f8(17.0, orc.IEEE) == f8(16.0, orc.IEEE)  # tie to even
    assert f8(19.0, orc.IEEE) == f8(20.0, orc.IEEE)


def test_against_compiled_reference_on_fresh_inputs(orc):
    R = orc.ref()
    if R is None:
        pytest.skip("oracle/_ref is not built here (the reference tree is absent)")
    import ctypes
    g = np.random.Generator(np.random.PCG64(99))
    x = g.integers(0, 2**32, 400000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    vp = ctypes.c_void_p
    for fn, dt, odt in ((R.ref_f32_to_f8e4m3fn_bulk, np.uint8, orc.F8E4M3FN), (R.ref_f32_to_f16_bulk, np.uint16, orc.F16),
                        (R.ref_f32_to_bf16_bulk, np.uint16, orc.BF16)):
        out = np.empty(x.size, dtype=dt)
        fn(x.ctypes.data_as(vp), out.ctypes.data_as(vp), x.size)
        assert np.array_equal(orc.narrow(x, odt, orc.REFHOST), out)


def test_ieee_f16_equals_numpy(orc):
    g = np.random.Generator(np.random.PCG64(5))
    x = np.concatenate([g.integers(0, 2**32, 1 << 20, dtype=np.uint64).astype(np.uint32).view(np.float32),
                        _load("lowp_f32_samples.npz")["x_bits"].view(np.float32)])
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        expect = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(orc.narrow(x, orc.F16, orc.IEEE), expect)
    h = np.arange(65536, dtype=np.uint16)
    keep = ~np.isnan(h.view(np.float16))
    assert np.array_equal(orc.widen(h, orc.F16)[keep], h.view(np.float16).astype(np.float32)[keep])


def test_ieee_bf16_and_f8_equal_torch(orc):
    import torch
    g = np.random.Generator(np.random.PCG64(6))
    x = np.concatenate([g.integers(0, 2**32, 1 << 20, dtype=np.uint64).astype(np.uint32).view(np.float32),
                        _load("lowp_f32_samples.npz")["x_bits"].view(np.float32)])
    x = x[np.isfinite(x)]
    t = torch.from_numpy(x.copy())
    expect = t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(orc.narrow(x, orc.BF16, orc.IEEE), expect)
    # torch's float8_e4m3fn cast rounds to nearest even and maps overflow to NaN, not to 448:
    # compare inside the finite range, where the two definitions coincide
    xin = x[np.abs(x) <= 448.0]
    e8 = torch.from_numpy(xin.copy()).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(orc.narrow(xin, orc.F8E4M3FN, orc.IEEE), e8)
    assert np.all(orc.narrow(np.float32([449, 464, 465, 1e9, np.inf]), orc.F8E4M3FN, orc.IEEE) == 0x7E)
    assert np.all(orc.narrow(np.float32([-465, -np.inf]), orc.F8E4M3FN, orc.IEEE) == 0xFE)
    codes = np.arange(256, dtype=np.uint8)
    back = torch.from_numpy(codes.copy()).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    ok = ~np.isnan(back)
    assert np.array_equal(orc.widen(codes, orc.F8E4M3FN)[ok], back[ok])


def test_reference_known_answers(orc):
    ka = json.load(open(os.path.join(GOLD, "reference_known_answers.json")))
    L = orc.lib()
    for mode in (orc.IEEE, orc.REFHOST):
        for case in ka["f32_to_f8"]:
            got = L.orc_f8e4m3fn_to_f32(L.orc_f32_to_f8e4m3fn(np.float32(case["x"]), mode))
            assert got == case["y"], (case, mode)
        for case in ka["f8_raw"]:
            assert L.orc_f32_to_f8e4m3fn(float(case["x"]), mode) == case["bits"], (case, mode)
        for case in ka["f32_to_bf16"]:
            got = L.orc_bf16_to_f32(L.orc_f32_to_bf16(np.float32(case["x"]), mode))
            assert got == case["y"], (case, mode)
    for case in ka["fptosi_f32_i4"]:
        assert L.orc_int4_saturate(int(math.trunc(case["x"]))) == case["y"]
    for case in ka["int4"]:
        if case["op"] == "zext":
            assert (L.orc_int4_saturate(case["x"]) & 0xF) == case["y"]
        elif case["op"] == "sext":
            assert L.orc_int4_sign_extend(L.orc_int4_saturate(case["x"]) & 0xF) == case["y"]
        elif case["op"] == "wrap_add":
            assert L.orc_int4_sign_extend((case["x"][0] + case["x"][1]) & 0xF) == case["y"]
        elif case["op"] == "pack":
            assert int(orc.pack_int4(np.int8(case["x"]))[0]) == case["y"]


def test_int4_pack_roundtrip(orc):
    v = np.arange(-8, 8, dtype=np.int8)
    v = np.concatenate([v, v[::-1], np.int8([3])])           # odd count: the last high nibble is zero
    p = orc.pack_int4(v)
    assert p.size == (v.size + 1) // 2 and (p[-1] >> 4) == 0
    assert np.array_equal(orc.unpack_int4(p, v.size), v)
    assert p[0] == ((-8 & 0xF) | ((-7 & 0xF) << 4))
