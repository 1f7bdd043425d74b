"""Host-side Python access to libmtrt_hip.so (ctypes, no torch types cross the ABI).

The directory name carries a hyphen, so the package is loaded by path under the
module name `tensorrt_incubator_amd` (see `__graft_entry__.load_package`).

torch is used only to own device memory and streams: every wrapper below passes
raw device pointers, extents and the current stream handle to the C ABI declared
in include/mtrt_hip.h.  There is no fallback: if the shared library is missing or
no gfx950 device is usable, the calls raise.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(_HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libmtrt_hip.so")
KERNEL_MODULE_PATH = os.path.join(LIB_DIR, "mtrt_kernels.hsaco")
FIXTURE_MODULE_PATH = os.path.join(LIB_DIR, "mtrt_test_fixtures.hsaco")

# enum mtrt_hip_dtype
F32, F16, BF16, I8, F8E4M3FN, I4, I4_PACKED = range(7)
F4_PACKED = 8
# enum mtrt_hip_scale_kind
SCALE_UNIFORM, SCALE_ROW, SCALE_COL = range(3)
# enum mtrt_hip_flags
Q_ROUND_TO_INT = 1
F8_REFHOST = 2
F8_VIA_F16 = 4

_c = ctypes
_vp, _i32, _i64, _f32, _sz, _i8 = _c.c_void_p, _c.c_int32, _c.c_int64, _c.c_float, _c.c_size_t, _c.c_int8

# name -> (restype, argtypes); mirrors include/mtrt_hip.h one to one
PROTOTYPES = {
    "mtrt_cuda_get_active_device": (_i32, []),
    "mtrt_cuda_set_active_device": (_i32, [_i32]),
    "mtrt_cuda_get_device": (_i32, [_i32]),
    "mtrt_cuda_get_device_count": (_i32, []),
    "mtrt_cuda_stream_create": (_vp, []),
    "mtrt_cuda_stream_destroy": (None, [_vp]),
    "mtrt_cuda_stream_sync": (None, [_vp]),
    "mtrt_cuda_event_create": (_vp, [_i32]),
    "mtrt_cuda_event_release": (None, [_vp]),
    "mtrt_cuda_stream_record_event": (None, [_vp, _vp]),
    "mtrt_cuda_stream_wait_event": (None, [_vp, _vp]),
    "mtrt_cuda_event_sync": (None, [_vp]),
    "mtrt_cuda_event_elapsed_msec": (_f32, [_vp, _vp]),
    "mtrt_cuda_alloc_async": (_vp, [_vp, _i64, _i32, _i8, _i8]),
    "mtrt_cuda_memcpy_async": (None, [_vp, _vp, _vp, _i64]),
    "mtrt_cuda_free": (None, [_vp, _vp, _i8, _i8]),
    "mtrt_cuda_module_load_from_ptx": (_vp, [_c.c_char_p, _sz]),
    "mtrt_cuda_module_load_from_ptx_file": (_vp, [_c.c_char_p, _sz]),
    "mtrt_cuda_module_unload": (None, [_vp]),
    "mtrt_cuda_module_get_function": (_vp, [_vp, _c.c_char_p, _i64]),
    "mtrt_cuda_launch_kernel": (None, [_vp, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _vp, _c.POINTER(_vp)]),
    "mtrt_cuda_get_current_device": (_i32, []),
    "mtrt_cuda_get_program_device": (_i32, [_i32]),
    # interpreter builtin bodies: handles travel as uintptr_t
    "mtrt_lua_cuda_load_module": (_i32, [_c.c_uint32, _sz, _c.c_uint64, _c.POINTER(_sz)]),
    "mtrt_lua_cuda_get_function": (_i32, [_sz, _c.c_char_p, _c.POINTER(_sz)]),
    "mtrt_lua_cuda_launch": (_i32, [_sz, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _sz, _sz]),
    "mtrt_lua_cuda_stream_create": (_i32, [_c.POINTER(_sz)]),
    "mtrt_lua_cuda_stream_sync": (_i32, [_sz]),
    "mtrt_lua_cuda_stream_destroy": (_i32, [_sz]),
    "mtrt_lua_cuda_alloc_device": (_i32, [_sz, _c.c_uint64, _c.POINTER(_sz)]),
    "mtrt_lua_cuda_free_device": (_i32, [_sz, _sz]),
    "mtrt_lua_cuda_memcpy": (_i32, [_sz, _sz, _c.c_uint64, _sz, _c.c_uint64, _c.c_uint64]),
    "mtrt_lua_cuda_memset": (_i32, [_sz, _sz, _c.c_uint64, _c.c_uint64, _c.c_uint32, _i32]),
    "mtrt_lua_cuda_event_create": (_i32, [_i32, _c.POINTER(_sz)]),
    "mtrt_lua_cuda_event_release": (_i32, [_sz]),
    "mtrt_lua_cuda_stream_record_event": (_i32, [_sz, _sz]),
    "mtrt_lua_cuda_stream_wait_event": (_i32, [_sz, _sz]),
    "mtrt_lua_cuda_event_sync": (_i32, [_sz]),
    "mtrt_lua_cuda_event_elapsed_msec": (_i32, [_sz, _sz, _c.POINTER(_f32)]),
    "mtrt_lua_cuda_alloc_host_pinned": (_i32, [_c.c_uint64, _i32, _c.POINTER(_sz)]),
    "mtrt_lua_cuda_free_host_pinned": (_i32, [_sz, _sz]),
    "mtrt_lua_cuda_memcpy_strided": (_i32, [_sz, _i64, _i64, _sz, _c.c_uint64, _c.POINTER(_i64), _sz, _c.c_uint64,
                                            _c.POINTER(_i64)]),
    "mtrt_lua_cuda_get_active_device": (_i32, [_c.POINTER(_i32)]),
    "mtrt_lua_cuda_set_active_device": (_i32, [_i32]),
    "mtrt_lua_cuda_get_device": (_i32, [_i32, _c.POINTER(_i32)]),
    "mtrt_lua_cuda_num_devices": (_i32, [_c.POINTER(_i32)]),
    "mtrt_lua_cuda_get_program_device": (_i32, [_i32, _c.POINTER(_i32)]),
    "mtrt_lua_cuda_builtins": (_vp, [_c.POINTER(_sz)]),
    "mtrt_hip_last_error": (_c.c_char_p, []),
    "mtrt_hip_last_kernel": (_c.c_char_p, []),
    "mtrt_hip_init": (_i32, []),
    "mtrt_hip_builtin_module": (_vp, []),
    "mtrt_hip_builtin_code_object": (_vp, [_c.POINTER(_sz)]),
    "mtrt_hip_amax": (_i32, [_vp, _vp, _i32, _i64, _f32, _vp, _vp]),
    "mtrt_hip_amax_scales": (_i32, [_vp, _vp, _i32, _i32, _i64, _i64, _i64, _f32, _vp, _vp]),
    "mtrt_hip_reset_reductions": (_i32, [_vp]),
    "mtrt_hip_amax_no_alloc": (_i32, [_vp, _vp, _i32, _i64, _f32, _vp, _vp]),
    "mtrt_hip_quantize": (_i32, [_vp, _vp, _i32, _vp, _i32, _vp, _i32, _i64, _i64, _i64, _i32]),
    "mtrt_hip_dequantize": (_i32, [_vp, _vp, _i32, _vp, _i32, _vp, _i32, _i64, _i64, _i64]),
    "mtrt_hip_quantize_dequantize": (_i32, [_vp, _vp, _i32, _vp, _i32, _vp, _vp, _i32, _i64, _i64, _i64, _i32]),
    "mtrt_hip_dynamic_quantize_dequantize": (_i32, [_vp, _vp, _i32, _vp, _i32, _vp, _i64, _f32, _vp, _vp, _i32]),
    "mtrt_hip_dynamic_quantize_rows": (_i32, [_vp, _vp, _i32, _vp, _i32, _i64, _i64, _f32, _vp, _vp, _i32]),
    "mtrt_hip_set_wait_limit": (_i32, [_i32]),
    "mtrt_hip_quantize_view": (_i32, [_vp, _vp, _i32, _vp, _vp, _i32, _vp, _vp, _i32, _i64, _i64, _i64, _i32]),
    "mtrt_hip_dequantize_view": (_i32, [_vp, _vp, _i32, _vp, _vp, _i32, _vp, _vp, _i32, _i64, _i64, _i64]),
    "mtrt_hip_nvfp4_quantize": (_i32, [_vp, _vp, _i32, _vp, _vp, _vp, _i64, _i64, _i32]),
    "mtrt_hip_nvfp4_dequantize": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i64, _i64, _i32]),
    "mtrt_hip_layernorm": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i64, _i64, _f32]),
    "mtrt_hip_softmax": (_i32, [_vp, _vp, _vp, _i32, _i64, _i64]),
    "mtrt_hip_gemm_w8a8_prepack": (_i32, [_vp, _vp, _vp, _i64, _i64]),
    "mtrt_hip_gemm_w8a8": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64]),
    "mtrt_hip_gemm_w8a8_fragments_bytes": (_i64, [_i64, _i64]),
    "mtrt_hip_gemm_w8a8_prepack_fragments": (_i32, [_vp, _vp, _i32, _vp, _i64, _i64]),
    "mtrt_hip_gemm_w8a8_fragments": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64]),
    "mtrt_hip_linear_dense": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i64, _i64, _i64]),
    "mtrt_hip_gemm_w4a16_prepacked_bytes": (_i64, [_i64, _i64]),
    "mtrt_hip_gemm_w4a16_prepack": (_i32, [_vp, _vp, _vp, _i64, _i64]),
    "mtrt_hip_gemm_w4a16": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64]),
}

_lib = None


class MtrtHipError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("mtrt_hip status %d: %s" % (code, message))
        self.code = code
        self.message = message


def lib():
    """The loaded C-ABI library with prototypes applied; raises if it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "%s is missing: run `python tensorrt-incubator_amd/build.py` (there is no fallback path)" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(status):
    if status != 0:
        raise MtrtHipError(status, lib().mtrt_hip_last_error().decode())


def last_kernel():
    return lib().mtrt_hip_last_kernel().decode()


# --------------------------------------------------------------------------
# torch-tensor conveniences (device memory + stream plumbing only)
# --------------------------------------------------------------------------

def _torch():
    import torch
    return torch


def float_dtype_of(t):
    torch = _torch()
    return {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}[t.dtype]


def _stream():
    return _torch().cuda.current_stream().cuda_stream


def _ptr(t):
    return None if t is None else t.data_ptr()


def code_tensor(q_dtype, numel, device):
    """Uninitialised storage for `numel` quantized codes (uint8/int8 bytes)."""
    torch = _torch()
    if q_dtype == I8:
        return torch.empty(numel, dtype=torch.int8, device=device)
    if q_dtype in (I4_PACKED, F4_PACKED):
        return torch.empty((numel + 1) // 2, dtype=torch.uint8, device=device)
    return torch.empty(numel, dtype=torch.uint8, device=device)


def amax(x, qmax):
    """Returns (amax, scale) as two 0-d f32 device tensors; scale = amax / qmax."""
    torch = _torch()
    assert x.is_cuda and x.is_contiguous()
    out = torch.empty(2, dtype=torch.float32, device=x.device)
    check(lib().mtrt_hip_amax(_stream(), x.data_ptr(), float_dtype_of(x), x.numel(), float(qmax),
                              out.data_ptr(), out.data_ptr() + 4))
    return out[0], out[1]


def amax_scales(x, qmax, kind, d0=None, d1=None, nb=1):
    """(amax, scale) f32 device tensors with one element per scale element of the addressing (kind, nb) over the
    [d0, d1] view of x: nb elements for SCALE_ROW, (d0 / nb) * d1 for SCALE_COL, one for SCALE_UNIFORM."""
    torch = _torch()
    assert x.is_cuda and x.is_contiguous()
    d0, d1 = _view2d(x, d0, d1)
    count = 1 if kind == SCALE_UNIFORM else (nb if kind == SCALE_ROW else (d0 // nb) * d1)
    out = torch.empty((2, max(count, 0)), dtype=torch.float32, device=x.device)
    check(lib().mtrt_hip_amax_scales(_stream(), x.data_ptr(), float_dtype_of(x), kind, d0, d1, nb, float(qmax),
                                     out[0].data_ptr(), out[1].data_ptr()))
    return out[0], out[1]


def quantize(x, scale, q_dtype, kind=SCALE_UNIFORM, d0=None, d1=None, nb=1, flags=0, out=None):
    assert x.is_cuda and x.is_contiguous() and scale.is_cuda and scale.dtype == _torch().float32
    d0, d1 = _view2d(x, d0, d1)
    q = code_tensor(q_dtype, d0 * d1, x.device) if out is None else out
    check(lib().mtrt_hip_quantize(_stream(), x.data_ptr(), float_dtype_of(x), q.data_ptr(), q_dtype,
                                  scale.data_ptr(), kind, d0, d1, nb, flags))
    return q


def dequantize(q, scale, q_dtype, out_torch_dtype, shape, kind=SCALE_UNIFORM, d0=None, d1=None, nb=1, out=None):
    torch = _torch()
    assert q.is_cuda and q.is_contiguous() and scale.dtype == torch.float32
    y = torch.empty(shape, dtype=out_torch_dtype, device=q.device) if out is None else out
    d0, d1 = _view2d(y, d0, d1)
    check(lib().mtrt_hip_dequantize(_stream(), q.data_ptr(), q_dtype, y.data_ptr(), float_dtype_of(y),
                                    scale.data_ptr(), kind, d0, d1, nb))
    return y


def quantize_dequantize(x, scale, q_dtype, kind=SCALE_UNIFORM, d0=None, d1=None, nb=1, flags=0, q_out=None, y_out=None):
    torch = _torch()
    assert x.is_cuda and x.is_contiguous() and scale.dtype == torch.float32
    d0, d1 = _view2d(x, d0, d1)
    q = code_tensor(q_dtype, d0 * d1, x.device) if q_out is None else q_out
    y = torch.empty_like(x) if y_out is None else y_out
    check(lib().mtrt_hip_quantize_dequantize(_stream(), x.data_ptr(), float_dtype_of(x), q.data_ptr(), q_dtype,
                                             y.data_ptr(), scale.data_ptr(), kind, d0, d1, nb, flags))
    return q, y


def dynamic_quantize_dequantize(x, q_dtype, qmax, flags=0, dequantize=True):
    """amax -> scale -> quantize (-> dequantize) of the whole tensor in one call; returns (q, y or None, amax, scale)."""
    torch = _torch()
    assert x.is_cuda and x.is_contiguous()
    out = torch.empty(2, dtype=torch.float32, device=x.device)
    q = code_tensor(q_dtype, x.numel(), x.device)
    y = torch.empty_like(x) if dequantize else None
    check(lib().mtrt_hip_dynamic_quantize_dequantize(_stream(), x.data_ptr(), float_dtype_of(x), q.data_ptr(), q_dtype,
                                                     _ptr(y), x.numel(), float(qmax), out.data_ptr(), out.data_ptr() + 4,
                                                     flags))
    return q, y, out[0], out[1]


def dynamic_quantize_rows(x, q_dtype, qmax, flags=0, want_amax=True):
    """Per-row amax -> scale -> quantize of a [rows, d] tensor (leading axes folded into rows) in one call; returns
    (q [rows * d] codes, amax [rows] or None, scale [rows])."""
    torch = _torch()
    assert x.is_cuda and x.is_contiguous() and x.dim() >= 1
    d = x.shape[-1]
    rows = x.numel() // d if d else 0
    out = torch.empty((2, rows), dtype=torch.float32, device=x.device)
    q = code_tensor(q_dtype, x.numel(), x.device)
    check(lib().mtrt_hip_dynamic_quantize_rows(_stream(), x.data_ptr(), float_dtype_of(x), q.data_ptr(), q_dtype, rows, d,
                                               float(qmax), out[0].data_ptr() if want_amax else None, out[1].data_ptr(), flags))
    return q, (out[0] if want_amax else None), out[1]


class View2d(ctypes.Structure):
    """struct mtrt_hip_view2d"""
    _fields_ = [("offset", _i64), ("stride0", _i64), ("stride1", _i64)]


def _view_of(t):
    """(base pointer of the storage, View2d) of a rank-2 torch view."""
    assert t.dim() == 2
    base = t.data_ptr() - t.storage_offset() * t.element_size()
    return base, View2d(t.storage_offset(), t.stride(0), t.stride(1))


def quantize_view(x, scale, q_dtype, q_out, kind=SCALE_UNIFORM, nb=1, flags=0):
    """Quantize the rank-2 view `x` (any strides) into the rank-2 view `q_out` (int8 / uint8 storage, any strides)."""
    assert x.is_cuda and q_out.is_cuda and tuple(x.shape) == tuple(q_out.shape) and scale.dtype == _torch().float32
    xb, xv = _view_of(x)
    qb, qv = _view_of(q_out)
    check(lib().mtrt_hip_quantize_view(_stream(), xb, float_dtype_of(x), ctypes.byref(xv), qb, q_dtype, ctypes.byref(qv),
                                       scale.data_ptr(), kind, x.shape[0], x.shape[1], nb, flags))
    return q_out


def dequantize_view(q, scale, q_dtype, y_out, kind=SCALE_UNIFORM, nb=1):
    assert q.is_cuda and y_out.is_cuda and tuple(q.shape) == tuple(y_out.shape) and scale.dtype == _torch().float32
    qb, qv = _view_of(q)
    yb, yv = _view_of(y_out)
    check(lib().mtrt_hip_dequantize_view(_stream(), qb, q_dtype, ctypes.byref(qv), yb, float_dtype_of(y_out), ctypes.byref(yv),
                                         scale.data_ptr(), kind, q.shape[0], q.shape[1], nb))
    return y_out


def nvfp4_quantize(x, tensor_amax, axis=-1):
    """NVFP4 codes (uint8, two per byte) and block scales (uint8 f8e4m3fn bytes, the shape of `x` with the blocked
    extent divided by 16) of `x`, blocks of 16 along `axis` (-1 or -2); `tensor_amax` is a 0-d f32 device
    tensor (what amax() returns)."""
    torch = _torch()
    assert x.is_cuda and x.is_contiguous() and tensor_amax.is_cuda and tensor_amax.dtype == torch.float32
    assert axis in (-1, -2, x.dim() - 1, x.dim() - 2)
    last = axis in (-1, x.dim() - 1)
    d1 = x.shape[-1]
    d0 = x.numel() // d1 if d1 else 0
    q = torch.empty(x.numel() // 2, dtype=torch.uint8, device=x.device)
    sshape = x.shape[:-1] + (d1 // 16,) if last else x.shape[:-2] + (x.shape[-2] // 16, d1)
    s = torch.empty(sshape, dtype=torch.uint8, device=x.device)
    check(lib().mtrt_hip_nvfp4_quantize(_stream(), x.data_ptr(), float_dtype_of(x), q.data_ptr(), s.data_ptr(),
                                        tensor_amax.data_ptr(), d0, d1, 1 if last else 0))
    return q, s


def nvfp4_dequantize(q, scales, tensor_amax, out_torch_dtype, shape, axis=-1):
    torch = _torch()
    assert q.is_cuda and q.dtype == torch.uint8 and scales.dtype == torch.uint8 and tensor_amax.dtype == torch.float32
    y = torch.empty(shape, dtype=out_torch_dtype, device=q.device)
    last = axis in (-1, y.dim() - 1)
    d1 = y.shape[-1]
    d0 = y.numel() // d1 if d1 else 0
    check(lib().mtrt_hip_nvfp4_dequantize(_stream(), q.data_ptr(), scales.data_ptr(), tensor_amax.data_ptr(),
                                          y.data_ptr(), float_dtype_of(y), d0, d1, 1 if last else 0))
    return y


def layernorm(x, gamma, beta, eps, out=None):
    torch = _torch()
    assert x.is_cuda and x.is_contiguous() and gamma.dtype == x.dtype and beta.dtype == x.dtype
    d = x.shape[-1]
    rows = x.numel() // d if d else 0
    y = torch.empty_like(x) if out is None else out
    check(lib().mtrt_hip_layernorm(_stream(), x.data_ptr(), gamma.data_ptr(), beta.data_ptr(), y.data_ptr(),
                                   float_dtype_of(x), rows, d, float(eps)))
    return y


def softmax(x, out=None):
    torch = _torch()
    assert x.is_cuda and x.is_contiguous()
    d = x.shape[-1]
    rows = x.numel() // d if d else 0
    y = torch.empty_like(x) if out is None else out
    check(lib().mtrt_hip_softmax(_stream(), x.data_ptr(), y.data_ptr(), float_dtype_of(x), rows, d))
    return y


def gemm_w8a8_prepack(w_kn):
    """int8 weights [K,N] -> [N,K] (the layout the GEMM consumes)."""
    torch = _torch()
    assert w_kn.is_cuda and w_kn.is_contiguous() and w_kn.dtype == torch.int8 and w_kn.dim() == 2
    K, N = w_kn.shape
    w_nk = torch.empty((N, K), dtype=torch.int8, device=w_kn.device)
    check(lib().mtrt_hip_gemm_w8a8_prepack(_stream(), w_kn.data_ptr(), w_nk.data_ptr(), K, N))
    return w_nk


def gemm_w8a8(a, w_nk, a_scale, w_scale, out=None):
    torch = _torch()
    assert a.is_cuda and a.is_contiguous() and a.dtype == torch.int8 and w_nk.is_contiguous() and w_nk.dtype == torch.int8
    assert a_scale.dtype == torch.float32 and w_scale.dtype == torch.float32
    M, K = a.shape
    N = w_nk.shape[0]
    assert w_nk.shape[1] == K and a_scale.numel() == M and w_scale.numel() == N
    y = torch.empty((M, N), dtype=torch.float16, device=a.device) if out is None else out
    check(lib().mtrt_hip_gemm_w8a8(_stream(), a.data_ptr(), w_nk.data_ptr(), a_scale.data_ptr(), w_scale.data_ptr(),
                                   y.data_ptr(), M, K, N))
    return y


def gemm_w8a8_prepack_fragments(w, is_nk=False):
    """int8 weights [K,N] (or [N,K] with is_nk) -> fragment-order buffer of the weights-in-registers kernel."""
    torch = _torch()
    assert w.is_cuda and w.is_contiguous() and w.dtype == torch.int8 and w.dim() == 2
    N, K = w.shape if is_nk else (w.shape[1], w.shape[0])
    nbytes = lib().mtrt_hip_gemm_w8a8_fragments_bytes(K, N)
    assert nbytes > 0, "fragment order needs K % 128 == 0"
    wf = torch.empty(nbytes, dtype=torch.int8, device=w.device)
    check(lib().mtrt_hip_gemm_w8a8_prepack_fragments(_stream(), w.data_ptr(), 1 if is_nk else 0, wf.data_ptr(), K, N))
    return wf


def gemm_w8a8_fragments(a, w_frag, a_scale, w_scale, N, out=None):
    torch = _torch()
    assert a.is_cuda and a.is_contiguous() and a.dtype == torch.int8 and w_frag.dtype == torch.int8
    assert a_scale.dtype == torch.float32 and w_scale.dtype == torch.float32
    M, K = a.shape
    assert a_scale.numel() == M and w_scale.numel() == N
    assert w_frag.numel() == lib().mtrt_hip_gemm_w8a8_fragments_bytes(K, N)
    y = torch.empty((M, N), dtype=torch.float16, device=a.device) if out is None else out
    check(lib().mtrt_hip_gemm_w8a8_fragments(_stream(), a.data_ptr(), w_frag.data_ptr(), a_scale.data_ptr(),
                                             w_scale.data_ptr(), y.data_ptr(), M, K, N))
    return y


def gemm_w4a16_prepack(w_kn_packed, K, N):
    """packed int4 weights (uint8, K*N/2 bytes over the flattened [K,N]) -> fragment-order buffer."""
    torch = _torch()
    assert w_kn_packed.is_cuda and w_kn_packed.is_contiguous() and w_kn_packed.dtype == torch.uint8
    nbytes = lib().mtrt_hip_gemm_w4a16_prepacked_bytes(K, N)
    assert nbytes > 0, "prepack needs K % 64 == 0"
    wp = torch.empty(nbytes, dtype=torch.uint8, device=w_kn_packed.device)
    check(lib().mtrt_hip_gemm_w4a16_prepack(_stream(), w_kn_packed.data_ptr(), wp.data_ptr(), K, N))
    return wp


def gemm_w4a16(a, scale, K, N, block, w_kn_packed=None, w_prepacked=None, out=None):
    torch = _torch()
    assert a.is_cuda and a.is_contiguous() and a.dtype == torch.float16 and scale.dtype == torch.float16
    M = a.shape[0]
    y = torch.empty((M, N), dtype=torch.float16, device=a.device) if out is None else out
    check(lib().mtrt_hip_gemm_w4a16(_stream(), a.data_ptr(), _ptr(w_kn_packed), _ptr(w_prepacked), scale.data_ptr(),
                                    y.data_ptr(), M, K, N, block))
    return y


def linear_dense(x, w_nk, bias=None, out=None):
    """y = x @ w_nk^T (+ bias) in the operands' float type, f32 accumulation; x [M,K], w_nk [N,K]."""
    torch = _torch()
    assert x.is_cuda and x.is_contiguous() and w_nk.is_contiguous() and w_nk.dtype == x.dtype and x.dim() == 2
    M, K = x.shape
    N = w_nk.shape[0]
    assert w_nk.shape[1] == K and (bias is None or (bias.dtype == x.dtype and bias.numel() == N and bias.is_contiguous()))
    y = torch.empty((M, N), dtype=x.dtype, device=x.device) if out is None else out
    check(lib().mtrt_hip_linear_dense(_stream(), x.data_ptr(), w_nk.data_ptr(), _ptr(bias), y.data_ptr(),
                                      float_dtype_of(x), M, K, N))
    return y


def _view2d(t, d0, d1):
    if d0 is None or d1 is None:
        if t.dim() == 0:
            return 1, 1
        d1 = t.shape[-1]
        d0 = t.numel() // d1 if d1 else 0
    return int(d0), int(d1)
