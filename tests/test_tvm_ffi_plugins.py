"""TVM-FFI plugin entry points of the library (`executor.call_plugin` boundary).

The argument arrays are built exactly as the reference's compiler emits them: a TVMFFIAny is
{i32 type_index, i32 0, i64 value}, a memref argument is type_index 7 with the address of a DLTensor
{data, {device_type 2, device_id}, ndim, {code, bits, lanes}, shape*, strides*, byte_offset}
(known answer: mlir-tensorrt/executor/test/Passes/executor-to-executor-plugin.mlir:30-62, f32 = code 2 bits 32
lanes 1).  The library-side convention (`__tvm_ffi_<name>` symbols, 0 / -1 return) is restated from
apache-tvm-ffi 0.1.3, which is absent: parity unpinned for that part."""
import ctypes

import numpy as np
import pytest


class Any(ctypes.Structure):
    class V(ctypes.Union):
        _fields_ = [("i", ctypes.c_int64), ("f", ctypes.c_double), ("p", ctypes.c_void_p)]
    _fields_ = [("type_index", ctypes.c_int32), ("zero_padding", ctypes.c_int32), ("v", V)]


class DLTensor(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("device_type", ctypes.c_int32), ("device_id", ctypes.c_int32),
                ("ndim", ctypes.c_int32), ("code", ctypes.c_uint8), ("bits", ctypes.c_uint8), ("lanes", ctypes.c_uint16),
                ("shape", ctypes.POINTER(ctypes.c_int64)), ("strides", ctypes.POINTER(ctypes.c_int64)),
                ("byte_offset", ctypes.c_uint64)]


NAMES = ["mtrt_quantize", "mtrt_dequantize", "mtrt_amax", "mtrt_layernorm", "mtrt_softmax", "mtrt_gemm_w8a8"]


def _fn(L, name):
    f = getattr(L, "__tvm_ffi_" + name)
    f.restype = ctypes.c_int
    f.argtypes = [ctypes.c_void_p, ctypes.POINTER(Any), ctypes.c_int32, ctypes.POINTER(Any)]
    return f


def _dl(t, keep):
    """torch tensor -> DLTensor as the reference encodes a device memref (device type 2, explicit strides)."""
    import torch
    code_bits = {torch.float32: (2, 32), torch.float16: (2, 16), torch.bfloat16: (4, 16), torch.int8: (0, 8),
                 torch.float8_e4m3fn: (10, 8), torch.uint8: (1, 8)}[t.dtype]
    shape = (ctypes.c_int64 * max(t.dim(), 1))(*t.shape)
    strides = (ctypes.c_int64 * max(t.dim(), 1))(*t.stride())
    d = DLTensor(t.data_ptr(), 2, 0, t.dim(), code_bits[0], code_bits[1], 1, shape, strides, 0)
    keep += [shape, strides, d, t]
    return d


def _args(*values):
    keep = []
    arr = (Any * len(values))()
    for i, v in enumerate(values):
        if v is None:
            arr[i].type_index = 0
        elif isinstance(v, bool):
            arr[i].type_index, arr[i].v.i = 2, int(v)
        elif isinstance(v, int):
            arr[i].type_index, arr[i].v.i = 1, v
        elif isinstance(v, float):
            arr[i].type_index, arr[i].v.f = 3, v
        else:
            d = _dl(v, keep)
            arr[i].type_index, arr[i].v.p = 7, ctypes.addressof(d)
    return arr, keep


def test_symbols_and_rejections_without_a_device(pkg):
    """Every declared plugin is exported under the `__tvm_ffi_` prefix; malformed calls return -1 with a message
    before any device work."""
    L = pkg.lib()
    text = open(pkg.LIB_PATH.replace("tensorrt-incubator_amd/lib/libmtrt_hip.so", "include/mtrt_hip_tvm_ffi.h")).read()
    for name in NAMES:
        assert "MTRT_TVM_FFI_DECLARE(%s);" % name in text
        _fn(L, name)
    res = Any()
    arr, _ = _args(1, 2)
    assert _fn(L, "mtrt_softmax")(None, arr, 2, ctypes.byref(res)) == -1
    assert b"argument 0 (x) must be a tensor" in L.mtrt_hip_last_error()
    assert _fn(L, "mtrt_quantize")(None, arr, 2, ctypes.byref(res)) == -1
    assert b"expects (input, scale, output [, axis])" in L.mtrt_hip_last_error()
    host = DLTensor(1024, 1, 0, 1, 2, 32, 1, (ctypes.c_int64 * 1)(4), None, 0)      # device type 1: host memory
    arr2 = (Any * 2)()
    for i in range(2):
        arr2[i].type_index, arr2[i].v.p = 7, ctypes.addressof(host)
    assert _fn(L, "mtrt_softmax")(None, arr2, 2, ctypes.byref(res)) == -1
    assert b"must live in GPU memory" in L.mtrt_hip_last_error()


@pytest.mark.gpu
def test_plugins_against_the_oracle_and_the_cluster_entry_points(pkg, orc):
    """Each plugin is called through its exported symbol with the argument array the reference's compiler emits and
    its output is compared with the CPU oracle (bit for bit for amax, scales, codes, dequantized values and the int8
    GEMM) and, for the two tolerance-checked reductions, with the cluster entry point it forwards to."""
    import numpy as np
    import torch
    from helpers import bits16
    L = pkg.lib()
    torch.manual_seed(21)
    res = Any()

    def call(name, *values):
        arr, keep = _args(*values)
        rc = _fn(L, name)(None, arr, len(values), ctypes.byref(res))
        assert rc == 0, L.mtrt_hip_last_error()
        assert res.type_index == 0

    x = torch.randn(6, 40, 128, device="cuda").to(torch.bfloat16)
    # per-tensor fp8 through amax -> scale on the device
    both = torch.zeros(2, device="cuda")
    call("mtrt_amax", x, both, 448.0)
    amax, scale = pkg.amax(x, 448.0)
    assert torch.equal(both, torch.stack([amax.reshape(()), scale.reshape(())]))
    xs = bits16(x)
    amax_ref = orc.amax(xs, orc.BF16)
    scale_ref = orc.scale_from_amax(amax_ref, 448.0)
    assert both.cpu().numpy().tobytes() == np.array([amax_ref, scale_ref], dtype=np.float32).tobytes()
    q = torch.zeros(x.shape, dtype=torch.float8_e4m3fn, device="cuda")
    call("mtrt_quantize", x, both[1:], q)
    want_q = pkg.quantize(x, both[1:], pkg.F8E4M3FN)
    assert torch.equal(q.view(torch.uint8).ravel(), want_q.view(torch.uint8).ravel())
    q_ref = orc.quantize(xs, orc.BF16, orc.F8E4M3FN, [scale_ref], orc.SCALE_UNIFORM, 240, 128)
    assert np.array_equal(q.view(torch.uint8).cpu().numpy().ravel(), q_ref)
    y = torch.zeros_like(x)
    call("mtrt_dequantize", q, both[1:], y, None)
    want_y = pkg.dequantize(want_q, both[1:], pkg.F8E4M3FN, torch.bfloat16, x.shape)
    assert torch.equal(y.view(torch.int16), want_y.view(torch.int16).reshape(y.shape))
    assert np.array_equal(bits16(y), orc.dequantize(q_ref, orc.F8E4M3FN, orc.BF16, [scale_ref], orc.SCALE_UNIFORM, 240, 128))
    # per-channel int8 on the middle axis (scale[row % 40] over [240, 128]) and on the last axis
    s_mid = (torch.rand(40, device="cuda") * 0.05 + 0.01)
    q8 = torch.zeros(x.shape, dtype=torch.int8, device="cuda")
    call("mtrt_quantize", x, s_mid, q8, 1)
    want = pkg.quantize(x, s_mid, pkg.I8, pkg.SCALE_ROW, 240, 128, 40)
    assert torch.equal(q8.ravel(), want.ravel())
    assert np.array_equal(q8.cpu().numpy().ravel(),
                          orc.quantize(xs, orc.BF16, orc.I8, s_mid.cpu().numpy(), orc.SCALE_ROW, 240, 128, 40))
    s_last = (torch.rand(128, device="cuda") * 0.05 + 0.01)
    call("mtrt_quantize", x, s_last, q8, 2)
    want = pkg.quantize(x, s_last, pkg.I8, pkg.SCALE_COL, 240, 128, 240)
    assert torch.equal(q8.ravel(), want.ravel())
    assert np.array_equal(q8.cpu().numpy().ravel(),
                          orc.quantize(xs, orc.BF16, orc.I8, s_last.cpu().numpy(), orc.SCALE_COL, 240, 128, 240))
    # block scale along the second-to-last axis: [6, 40, 128] with scale [6, 5, 128] (blocks of 8 rows)
    s_blk = (torch.rand(6, 5, 128, device="cuda") * 0.05 + 0.01)
    xb = x[0].contiguous()                                  # [40, 128] with scale [5, 128]
    qb = torch.zeros(xb.shape, dtype=torch.int8, device="cuda")
    call("mtrt_quantize", xb, s_blk[0].contiguous(), qb)
    want = pkg.quantize(xb, s_blk[0].contiguous(), pkg.I8, pkg.SCALE_COL, 40, 128, 8)
    assert torch.equal(qb.ravel(), want.ravel())
    assert np.array_equal(qb.cpu().numpy().ravel(),
                          orc.quantize(bits16(xb), orc.BF16, orc.I8, s_blk[0].cpu().numpy().ravel(), orc.SCALE_COL, 40, 128, 8))
    # fused reduce clusters
    g = (torch.rand(128, device="cuda") + 0.5).to(torch.bfloat16)
    b = (torch.randn(128, device="cuda") * 0.1).to(torch.bfloat16)
    out = torch.zeros_like(x)
    call("mtrt_layernorm", x, g, b, out, 1e-5)
    assert torch.equal(out.view(torch.int16), pkg.layernorm(x, g, b, 1e-5).view(torch.int16))
    ln_ref = orc.widen(orc.layernorm(xs, bits16(g), bits16(b), orc.BF16, 240, 128, 1e-5), orc.BF16)
    assert np.max(np.abs(orc.widen(bits16(out), orc.BF16) - ln_ref) / (np.abs(ln_ref) + 0.1)) <= 2.0 ** -7   # one bf16 ulp
    call("mtrt_softmax", x, out)
    assert torch.equal(out.view(torch.int16), pkg.softmax(x).view(torch.int16))
    sm_ref = orc.widen(orc.softmax(xs, orc.BF16, 240, 128), orc.BF16)
    assert np.max(np.abs(orc.widen(bits16(out), orc.BF16) - sm_ref) / (sm_ref + 1e-6)) <= 2.0 ** -7
    # int8 GEMM
    M, K, N = 96, 256, 160
    a = torch.randint(-128, 128, (M, K), dtype=torch.int8, device="cuda")
    w = torch.randint(-128, 128, (N, K), dtype=torch.int8, device="cuda")
    a_s, w_s = torch.rand(M, device="cuda") * 0.02, torch.rand(N, device="cuda") * 0.02
    yg = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    call("mtrt_gemm_w8a8", a, w, a_s, w_s, yg)
    assert torch.equal(yg.view(torch.int16), pkg.gemm_w8a8(a, w, a_s, w_s).view(torch.int16))
    y_ref = orc.gemm_w8a8(a.cpu().numpy(), np.ascontiguousarray(w.cpu().numpy().T), a_s.cpu().numpy(), w_s.cpu().numpy())
    assert np.array_equal(bits16(yg).reshape(M, N), y_ref)
    # a failing cluster call surfaces as -1 with the cluster's message
    arr, keep = _args(x, torch.zeros(3, device="cuda"), q)       # 3 scale elements fit no mode
    assert _fn(L, "mtrt_quantize")(None, arr, 3, ctypes.byref(res)) == -1
    assert b"scale must have one element" in L.mtrt_hip_last_error()
