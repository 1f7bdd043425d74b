"""TEST INFRASTRUCTURE — ctypes access to the CPU oracle (oracle/liboracle.so) and,
when it was built, to the compiled reference number classes (oracle/_ref).

Only tests, `__graft_entry__.smoke()` and the benchmark's cpu_baseline leg import
this module.  numpy arrays in, numpy arrays out; nothing here touches a GPU.
"""
import ctypes
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liboracle.so")
REF_PATH = os.path.join(HERE, "_ref", "libref_datatypes.so")

F32, F16, BF16, I8, F8E4M3FN, I4, I4_PACKED, I32, F4_PACKED = range(9)
IEEE, REFHOST = 0, 1
F8_VIA_F16 = 4
SCALE_UNIFORM, SCALE_ROW, SCALE_COL = range(3)
Q_ROUND_TO_INT = 1

_c = ctypes
_vp, _i32, _i64, _f32 = _c.c_void_p, _c.c_int32, _c.c_int64, _c.c_float
_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: run `make -C oracle`" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        L.orc_f32_to_f8e4m3fn.restype, L.orc_f32_to_f8e4m3fn.argtypes = _c.c_uint8, [_f32, _i32]
        L.orc_f8e4m3fn_to_f32.restype, L.orc_f8e4m3fn_to_f32.argtypes = _f32, [_c.c_uint8]
        L.orc_f32_to_f16.restype, L.orc_f32_to_f16.argtypes = _c.c_uint16, [_f32, _i32]
        L.orc_f16_to_f32.restype, L.orc_f16_to_f32.argtypes = _f32, [_c.c_uint16]
        L.orc_f32_to_bf16.restype, L.orc_f32_to_bf16.argtypes = _c.c_uint16, [_f32, _i32]
        L.orc_bf16_to_f32.restype, L.orc_bf16_to_f32.argtypes = _f32, [_c.c_uint16]
        L.orc_int4_saturate.restype, L.orc_int4_saturate.argtypes = _c.c_int8, [_i32]
        L.orc_int4_sign_extend.restype, L.orc_int4_sign_extend.argtypes = _c.c_int8, [_c.c_uint8]
        L.orc_narrow.restype, L.orc_narrow.argtypes = None, [_vp, _vp, _i32, _i64, _i32]
        L.orc_widen.restype, L.orc_widen.argtypes = None, [_vp, _i32, _vp, _i64]
        L.orc_pack_int4.restype, L.orc_pack_int4.argtypes = None, [_vp, _vp, _i64]
        L.orc_unpack_int4.restype, L.orc_unpack_int4.argtypes = None, [_vp, _vp, _i64]
        L.orc_amax.restype, L.orc_amax.argtypes = _f32, [_vp, _i32, _i64]
        L.orc_scale_from_amax.restype, L.orc_scale_from_amax.argtypes = _f32, [_f32, _f32]
        L.orc_amax_scales.restype = None
        L.orc_amax_scales.argtypes = [_vp, _i32, _i32, _i64, _i64, _i64, _f32, _vp, _vp]
        L.orc_quantize.restype = None
        L.orc_quantize.argtypes = [_vp, _i32, _vp, _i32, _vp, _i32, _i64, _i64, _i64, _i32, _i32]
        L.orc_dequantize.restype = None
        L.orc_dequantize.argtypes = [_vp, _i32, _vp, _i32, _vp, _i32, _i64, _i64, _i64, _i32]
        L.orc_layernorm.restype = None
        L.orc_layernorm.argtypes = [_vp, _vp, _vp, _vp, _i32, _i64, _i64, _f32, _i32]
        L.orc_softmax.restype, L.orc_softmax.argtypes = None, [_vp, _vp, _i32, _i64, _i64, _i32]
        L.orc_gemm_i8_i32.restype, L.orc_gemm_i8_i32.argtypes = None, [_vp, _vp, _vp, _i64, _i64, _i64]
        L.orc_gemm_w8a8.restype = None
        L.orc_gemm_w8a8.argtypes = [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i32]
        L.orc_gemm_w4a16.restype = None
        L.orc_gemm_w4a16.argtypes = [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i32]
        L.orc_f16_to_f4e2m1fn.restype, L.orc_f16_to_f4e2m1fn.argtypes = _c.c_uint8, [_c.c_uint16, _i32]
        L.orc_f4e2m1fn_to_f32.restype, L.orc_f4e2m1fn_to_f32.argtypes = _f32, [_c.c_uint8]
        L.orc_nvfp4_quantize.restype = None
        L.orc_nvfp4_quantize.argtypes = [_vp, _i32, _vp, _vp, _f32, _i64, _i64, _i32, _i32]
        L.orc_nvfp4_dequantize.restype = None
        L.orc_nvfp4_dequantize.argtypes = [_vp, _vp, _f32, _vp, _i32, _i64, _i64, _i32, _i32]
        _lib = L
    return _lib


def set_threads(n):
    """OpenMP threads used by the oracle loops (1 = faithful to the single-threaded interpreter)."""
    omp = ctypes.CDLL("libgomp.so.1")
    omp.omp_set_num_threads(int(n))


def ref():
    """The compiled reference number classes, or None where they were not built."""
    global _ref
    if _ref is None and os.path.exists(REF_PATH):
        R = ctypes.CDLL(REF_PATH)
        R.ref_f32_to_f8e4m3fn.restype, R.ref_f32_to_f8e4m3fn.argtypes = _c.c_uint8, [_f32]
        R.ref_f8e4m3fn_to_f32.restype, R.ref_f8e4m3fn_to_f32.argtypes = _f32, [_c.c_uint8]
        R.ref_f32_to_f16.restype, R.ref_f32_to_f16.argtypes = _c.c_uint16, [_f32]
        R.ref_f16_to_f32.restype, R.ref_f16_to_f32.argtypes = _f32, [_c.c_uint16]
        R.ref_f32_to_bf16.restype, R.ref_f32_to_bf16.argtypes = _c.c_uint16, [_f32]
        R.ref_bf16_to_f32.restype, R.ref_bf16_to_f32.argtypes = _f32, [_c.c_uint16]
        R.ref_int4_from_int.restype, R.ref_int4_from_int.argtypes = _c.c_int8, [_i32]
        R.ref_int4_raw_from_int.restype, R.ref_int4_raw_from_int.argtypes = _c.c_uint8, [_i32]
        R.ref_int4_from_raw.restype, R.ref_int4_from_raw.argtypes = _c.c_int8, [_c.c_uint8]
        R.ref_fptosi_f32_i4.restype, R.ref_fptosi_f32_i4.argtypes = _c.c_int8, [_f32]
        for n in ("ref_f32_to_f8e4m3fn_bulk", "ref_f32_to_f16_bulk", "ref_f32_to_bf16_bulk"):
            getattr(R, n).restype = None
            getattr(R, n).argtypes = [_vp, _vp, _i64]
        _ref = R
    return _ref


_NP_OF = {F32: np.float32, F16: np.uint16, BF16: np.uint16, I8: np.int8, F8E4M3FN: np.uint8, I4: np.uint8,
          I4_PACKED: np.uint8, I32: np.int32, F4_PACKED: np.uint8}


def _p(a):
    return a.ctypes.data_as(_vp)


def _c_arr(a, dtype):
    a = np.ascontiguousarray(a)
    assert a.dtype == _NP_OF[dtype], (a.dtype, dtype)
    return a


def storage_count(dtype, n):
    return (n + 1) // 2 if dtype in (I4_PACKED, F4_PACKED) else n


def narrow(x_f32, dst_dtype, mode=IEEE):
    x = np.ascontiguousarray(x_f32, dtype=np.float32)
    out = np.empty(x.shape, dtype=_NP_OF[dst_dtype])
    lib().orc_narrow(_p(x), _p(out), dst_dtype, x.size, mode)
    return out


def widen(a, src_dtype, n=None):
    a = _c_arr(a, src_dtype)
    n = a.size if n is None else n
    out = np.empty(n, dtype=np.float32)
    lib().orc_widen(_p(a), src_dtype, _p(out), n)
    return out.reshape(a.shape) if n == a.size else out


def pack_int4(unpacked_i8):
    u = np.ascontiguousarray(unpacked_i8, dtype=np.int8).ravel()
    out = np.empty((u.size + 1) // 2, dtype=np.uint8)
    lib().orc_pack_int4(_p(u), _p(out), u.size)
    return out


def unpack_int4(packed_u8, n):
    pk = np.ascontiguousarray(packed_u8, dtype=np.uint8).ravel()
    out = np.empty(n, dtype=np.int8)
    lib().orc_unpack_int4(_p(pk), _p(out), n)
    return out


def amax(x, dtype):
    x = _c_arr(x, dtype)
    return np.float32(lib().orc_amax(_p(x), dtype, x.size))


def scale_from_amax(amax_value, qmax):
    return np.float32(lib().orc_scale_from_amax(float(amax_value), float(qmax)))


def amax_scales(x, dtype, kind, d0, d1, nb, qmax):
    """(amax, scale) arrays, one element per scale element of the addressing (kind, nb)."""
    x = _c_arr(x, dtype)
    count = 1 if kind == SCALE_UNIFORM else (nb if kind == SCALE_ROW else (d0 // nb) * d1)
    amax = np.zeros(count, dtype=np.float32)
    scale = np.zeros(count, dtype=np.float32)
    lib().orc_amax_scales(_p(x), dtype, kind, d0, d1, nb, float(qmax), _p(amax), _p(scale))
    return amax, scale


def quantize(x, in_dtype, out_dtype, scale, kind, d0, d1, nb=1, flags=0, mode=IEEE):
    x = _c_arr(x, in_dtype)
    scale = np.ascontiguousarray(scale, dtype=np.float32)
    q = np.zeros(storage_count(out_dtype, d0 * d1), dtype=_NP_OF[out_dtype])
    lib().orc_quantize(_p(x), in_dtype, _p(q), out_dtype, _p(scale), kind, d0, d1, nb, flags, mode)
    return q


def dequantize(q, in_dtype, out_dtype, scale, kind, d0, d1, nb=1, mode=IEEE):
    q = _c_arr(q, in_dtype)
    scale = np.ascontiguousarray(scale, dtype=np.float32)
    y = np.empty(d0 * d1, dtype=_NP_OF[out_dtype])
    lib().orc_dequantize(_p(q), in_dtype, _p(y), out_dtype, _p(scale), kind, d0, d1, nb, mode)
    return y


def layernorm(x, gamma, beta, dtype, rows, d, eps, mode=IEEE):
    x, gamma, beta = _c_arr(x, dtype), _c_arr(gamma, dtype), _c_arr(beta, dtype)
    y = np.empty(rows * d, dtype=_NP_OF[dtype])
    lib().orc_layernorm(_p(x), _p(gamma), _p(beta), _p(y), dtype, rows, d, eps, mode)
    return y


def softmax(x, dtype, rows, d, mode=IEEE):
    x = _c_arr(x, dtype)
    y = np.empty(rows * d, dtype=_NP_OF[dtype])
    lib().orc_softmax(_p(x), _p(y), dtype, rows, d, mode)
    return y


def gemm_i8_i32(a, w):
    a, w = _c_arr(a, I8), _c_arr(w, I8)
    M, K = a.shape
    N = w.shape[1]
    acc = np.empty((M, N), dtype=np.int32)
    lib().orc_gemm_i8_i32(_p(a), _p(w), _p(acc), M, K, N)
    return acc


def gemm_w8a8(a, w, a_scale, w_scale, m0=0, mcount=None, mode=IEEE):
    a, w = _c_arr(a, I8), _c_arr(w, I8)
    M, K = a.shape
    N = w.shape[1]
    mcount = M - m0 if mcount is None else mcount
    a_scale = np.ascontiguousarray(a_scale, dtype=np.float32)
    w_scale = np.ascontiguousarray(w_scale, dtype=np.float32)
    y = np.zeros((M, N), dtype=np.uint16)
    lib().orc_gemm_w8a8(_p(a), _p(w), _p(a_scale), _p(w_scale), _p(y), M, K, N, m0, mcount, mode)
    return y[m0:m0 + mcount]


def gemm_w4a16(a_f16_bits, w_packed, scale_f16_bits, K, N, block, m0=0, mcount=None, mode=IEEE):
    a = _c_arr(a_f16_bits, F16)
    M = a.shape[0]
    mcount = M - m0 if mcount is None else mcount
    w = np.ascontiguousarray(w_packed, dtype=np.uint8)
    s = _c_arr(scale_f16_bits, F16)
    y = np.zeros((M, N), dtype=np.uint16)
    lib().orc_gemm_w4a16(_p(a), _p(w), _p(s), _p(y), M, K, N, block, m0, mcount, mode)
    return y[m0:m0 + mcount]


def nvfp4_quantize(x, in_dtype, tensor_amax, d0, d1, mode=IEEE, block_axis=1):
    """Returns (codes packed two per byte [d0*d1/2], block scales as f8e4m3fn bytes [d0*d1/16]);
    block_axis 1: blocks of 16 along d1, 0: along d0."""
    x = _c_arr(x, in_dtype)
    assert (d1 if block_axis else d0) % 16 == 0 and (d0 * d1) % 2 == 0
    q = np.zeros(d0 * d1 // 2, dtype=np.uint8)
    s = np.zeros(d0 * d1 // 16, dtype=np.uint8)
    lib().orc_nvfp4_quantize(_p(x), in_dtype, _p(q), _p(s), float(tensor_amax), d0, d1, block_axis, mode)
    return q, s


def nvfp4_dequantize(q, scales, tensor_amax, out_dtype, d0, d1, mode=IEEE, block_axis=1):
    q = np.ascontiguousarray(q, dtype=np.uint8)
    s = np.ascontiguousarray(scales, dtype=np.uint8)
    y = np.empty(d0 * d1, dtype=_NP_OF[out_dtype])
    lib().orc_nvfp4_dequantize(_p(q), _p(s), float(tensor_amax), _p(y), out_dtype, d0, d1, block_axis, mode)
    return y
