"""Values of the Tripy-compatible mirror on the GPU.

Known answers are those of the reference's integration tests:
  tripy/tests/integration/test_quantize.py:32-43, 58-69, 72-114, 121-145
  tripy/tests/integration/test_dequantize.py:30-79
  tripy/tests/integration/test_linear.py:54-130
  tripy/tests/integration/test_layernorm.py:24-109, test_softmax.py:18-40
  mlir-tensorrt/integrations/PJRT/test/JAX/CustomPrimitives/test_quantize.py:60-83
and, on seeded random data, the CPU oracle addressed independently of the mirror (the scale is
broadcast to the full shape with numpy and the oracle runs per-element on a flat view).
Bar: bit-exact codes and dequantized values; Linear within 1e-3 relative of a float64 product of
the oracle's dequantized operands.
"""
import importlib

import numpy as np
import pytest

from helpers import rng

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tp(pkg):
    return importlib.import_module(pkg.__name__ + ".tp")


def _torch_dtypes(tp):
    import torch
    return {tp.float32: torch.float32, tp.float16: torch.float16, tp.bfloat16: torch.bfloat16}


def _all_float(tp):
    return [tp.float32, tp.float16, tp.bfloat16]


def test_quantize_int8_per_tensor(tp):
    import torch
    for d in _all_float(tp):
        td = _torch_dtypes(tp)[d]
        x = torch.tensor([1.0, 2.0], dtype=td)
        scale = torch.tensor(0.5, dtype=td)
        q = tp.quantize(tp.Tensor(x), tp.Tensor(scale), tp.int8)
        assert q.dtype == tp.int8
        assert torch.equal((x / scale).to(torch.int8), q.torch().cpu())


def test_quantize_int8_per_channel(tp):
    import torch
    for d in (tp.float32, tp.bfloat16):
        td = _torch_dtypes(tp)[d]
        x = torch.tensor([[1.0, 2.0], [3.0, 4.0]], dtype=td)
        scale = torch.tensor([0.2, 0.1], dtype=td)
        q = tp.quantize(tp.Tensor(x), tp.Tensor(scale), tp.int8, dim=0)
        # the reference test truncates ((x/scale).to(int8)); the op rounds half to even
        # (TensorRTOps.td:3145-3185), which differs when the f32 quotient is not integral
        expected = torch.clamp(torch.round(x.float() / scale.float().reshape(2, 1)), -128, 127).to(torch.int8)
        assert torch.equal(expected, q.torch().cpu())


def test_quantize_float8(tp):
    import torch
    for d in _all_float(tp):
        td = _torch_dtypes(tp)[d]
        x = torch.tensor([1.0, 2.0], dtype=td)
        q = tp.quantize(tp.Tensor(x), tp.Tensor(torch.tensor(0.5, dtype=td)), tp.float8)
        assert q.dtype == tp.float8
        assert torch.equal(torch.tensor([2.0, 4.0]), tp.cast(q, tp.float32).torch().cpu())
        x2 = torch.tensor([[1.0, 2.0], [3.0, 4.0]], dtype=td)
        s2 = torch.tensor([0.5, 0.25], dtype=td)
        q2 = tp.quantize(tp.Tensor(x2), tp.Tensor(s2), tp.float8, dim=0)
        assert torch.equal(x2.float() / s2.float().reshape(2, 1), tp.cast(q2, tp.float32).torch().cpu())


@pytest.mark.parametrize("quant_mode", ["block-wise", "per-tensor", "per-channel-0", "per-channel-1"])
def test_qdq_int4(tp, quant_mode):
    import torch
    for d in _all_float(tp):
        td = _torch_dtypes(tp)[d]
        dim = None
        if quant_mode == "block-wise":
            scale = torch.ones((2, 4), dtype=td)
        elif quant_mode == "per-tensor":
            scale = torch.tensor(1.0, dtype=td)
        else:
            dim = int(quant_mode[-1])
            scale = torch.ones((4,), dtype=td)
        x = torch.ones((4, 4), dtype=td)
        s = tp.Tensor(scale)
        q = tp.quantize(tp.Tensor(x), s, tp.int4, dim)
        y = tp.dequantize(q, s, d, dim)
        assert y.dtype == d and torch.equal(x, y.torch().cpu())


def test_dequantize_int8(tp):
    import torch
    for d in _all_float(tp):
        td = _torch_dtypes(tp)[d]
        q = tp.cast(tp.Tensor([4, 8]), tp.int8)
        scale = torch.tensor(0.5, dtype=td)
        y = tp.dequantize(q, tp.Tensor(scale), d)
        assert torch.allclose(torch.tensor([4, 8]) * scale, y.torch().cpu())
        q2 = tp.cast(tp.Tensor([[4, 8], [4, 8]]), tp.int8)
        s2 = torch.tensor([0.8, 0.9], dtype=td)
        y2 = tp.dequantize(q2, tp.Tensor(s2), d, dim=0)
        assert torch.allclose(torch.tensor([[4, 8], [4, 8]]) * s2.reshape(2, 1), y2.torch().cpu())


def test_dequantize_float8_per_tensor(tp):
    import torch
    for d in _all_float(tp):
        td = _torch_dtypes(tp)[d]
        q = tp.cast(tp.Tensor([1.0, 1.0]), tp.float8)
        y = tp.dequantize(q, tp.Tensor(torch.tensor(0.5, dtype=td)), d)
        assert y.dtype == d
        assert torch.allclose(torch.tensor([0.5, 0.5]), y.torch().float().cpu())


def test_jax_custom_primitive_known_answers(tp):
    x = np.array([[10.0, 20.0, 30.0, 40.0], [50.0, 60.0, 70.0, 80.0]], dtype=np.float32)
    q = tp.quantize(tp.Tensor(x), 1.0, tp.int8)
    assert np.array_equal(q.torch().cpu().numpy(), x.astype(np.int8))
    q = tp.quantize(tp.Tensor(x), [2.0, 10.0], tp.int8, dim=0)
    assert np.array_equal(q.torch().cpu().numpy(), np.array([[5, 10, 15, 20], [5, 6, 7, 8]], dtype=np.int8))


def _oracle_elementwise(orc, x_f32, scale_full_f32, o_x, o_q):
    """Oracle result with the scale already broadcast: one row per element."""
    n = x_f32.size
    xs = orc.narrow(x_f32.ravel(), o_x)
    q = orc.quantize(xs, o_x, o_q, scale_full_f32.ravel(), orc.SCALE_ROW, n, 1, n)
    y = orc.dequantize(q, o_q, o_x, scale_full_f32.ravel(), orc.SCALE_ROW, n, 1, n)
    return xs, q, y


@pytest.mark.parametrize("case", [
    ("f32", "i8", (3, 5, 7), 1), ("bf16", "f8", (4, 6, 10), 2), ("f16", "i8", (6, 33), 0), ("f32", "i4", (5, 9, 4), 0),
    ("f32", "i8", (17, 64), None), ("bf16", "i4", (256, 48), "block"), ("f16", "f8", (2, 3, 4, 5), -1),
])
def test_modes_against_oracle(tp, orc, case):
    import torch
    xname, qname, shape, dim = case
    r = rng(1000 + sum(shape) * 7 + len(xname) + 3 * len(qname))
    d = {"f32": tp.float32, "f16": tp.float16, "bf16": tp.bfloat16}[xname]
    o_x = {"f32": orc.F32, "f16": orc.F16, "bf16": orc.BF16}[xname]
    qd, o_q, qmax = {"i8": (tp.int8, orc.I8, 127.0), "f8": (tp.float8, orc.F8E4M3FN, 448.0),
                     "i4": (tp.int4, orc.I4, 7.0)}[qname]
    x = (r.standard_normal(shape) * 3).astype(np.float32)
    if dim == "block":
        s = r.uniform(0.2, 1.5, (shape[0] // 64, shape[1])).astype(np.float32)
        full = np.repeat(s, 64, axis=0)
        dim_arg = None
    elif dim is None:
        s = np.float32(np.abs(x).max() / qmax)
        full = np.full(shape, s, dtype=np.float32)
        dim_arg = None
    else:
        c = shape[dim]
        s = r.uniform(0.01, 0.2, (c,)).astype(np.float32)
        view = [1] * len(shape)
        view[dim] = c
        full = np.broadcast_to(s.reshape(view), shape).astype(np.float32)
        dim_arg = dim
    # scale constants live in the input's type (the op requires scale.dtype == input.dtype)
    s_store = orc.widen(orc.narrow(np.asarray(s, dtype=np.float32).ravel(), o_x), o_x).reshape(np.shape(s))
    full_store = orc.widen(orc.narrow(full.ravel(), o_x), o_x).reshape(shape)
    xs, q_ref, y_ref = _oracle_elementwise(orc, x, full_store, o_x, o_q)

    td = _torch_dtypes(tp)[d]
    x_t = torch.from_numpy(orc.widen(xs, o_x).reshape(shape)).to(td)      # exact: values are representable
    s_t = torch.from_numpy(np.asarray(s_store, dtype=np.float32)).to(td)
    scale = tp.Tensor(s_t)
    q = tp.quantize(tp.Tensor(x_t), scale, qd, dim_arg)
    assert np.array_equal(q.torch().cpu().numpy().view(np.uint8).ravel(), q_ref.view(np.uint8).ravel())
    y = tp.dequantize(q, scale, d, dim_arg)
    got = y.torch().cpu()
    got_f32 = got.float().numpy().ravel()
    assert np.array_equal(got_f32.view(np.uint32), orc.widen(y_ref, o_x).view(np.uint32))


def test_quant_linear_reference_cases(tp):
    """tripy/tests/integration/test_linear.py:88-130: unit scales, small integers: exact."""
    import torch
    for quant_dtype in (tp.int8, tp.float8):
        for use_input_scale in (False, True):
            for wqd in (None, 0, 1):
                if use_input_scale and wqd == 1:
                    continue
                lin = tp.Linear(4, 2, quant_dtype=quant_dtype, weight_quant_dim=wqd)
                lin.weight = tp.iota((2, 4))
                lin.bias = tp.iota((2,))
                lin.weight_scale = tp.Tensor(1.0 if wqd is None else [1.0] * (2 if wqd == 0 else 4))
                if use_input_scale:
                    lin.input_scale = tp.Tensor(1.0)
                out = lin(tp.Tensor(np.ones((3, 4), dtype=np.float32)))
                w = lin.weight.torch().cpu().numpy()
                expect = np.ones((3, 4), dtype=np.float32) @ w.T + lin.bias.torch().cpu().numpy()
                assert np.array_equal(out.torch().cpu().numpy(), expect)
    for wqd, scale in [(None, np.ones((2, 4), dtype=np.float32)), (None, 1.0), (0, np.ones((8,), dtype=np.float32)),
                       (1, np.ones((4,), dtype=np.float32))]:
        lin = tp.Linear(4, 8, quant_dtype=tp.int4, weight_quant_dim=wqd)
        lin.weight_scale = tp.Tensor(scale)
        lin.weight = tp.Tensor(np.ones((8, 4), dtype=np.float32))
        lin.bias = tp.Tensor(np.ones((8,), dtype=np.float32))
        out = lin(tp.Tensor(np.ones((4, 4), dtype=np.float32)))
        assert np.array_equal(out.torch().cpu().numpy(), np.full((4, 8), 5.0, dtype=np.float32))


def test_quant_linear_int8_runs_on_the_w8a8_cluster(tp, orc, pkg):
    """int8 Linear in a float16 module with an input scale and per-output-channel weight scales lands on the integer
    matrix cores (fragment-order weights prepared once): against a float64 product of the oracle's dequantized
    operands, 1e-3 relative (f16 result)."""
    r = rng(77)
    for M, K, N, kernels in ((96, 256, 160, ("mtrt_gemm_w8a8_frag_rows128", "mtrt_gemm_w8a8_frag")), (5, 72, 33, ("mtrt_gemm_w8a8_nk_edge",))):
        x = r.standard_normal((M, K)).astype(np.float16)
        w = (r.standard_normal((N, K)) * 0.05).astype(np.float16)
        b = r.standard_normal(N).astype(np.float16)
        s_x = np.float16(np.abs(x.astype(np.float32)).max() / 127.0)
        s_w = (np.abs(w.astype(np.float32)).max(axis=1) / 127.0).astype(np.float16)
        lin = tp.Linear(K, N, dtype=tp.float16, quant_dtype=tp.int8, weight_quant_dim=0)
        lin.load_state_dict({"weight": tp.Tensor(w), "bias": tp.Tensor(b), "weight_scale": tp.Tensor(s_w),
                             "input_scale": tp.Tensor(s_x)})
        assert lin.route() == "w8a8"
        plan = lin._prepared()
        out = lin(tp.Tensor(x)).torch().cpu().numpy().astype(np.float64)
        assert lin._prepared() is plan, "the weight side must be prepared once, not per forward pass"
        assert pkg.last_kernel() in kernels

        s_x32, s_w32 = np.float32(s_x), s_w.astype(np.float32)
        qx = orc.quantize(x.view(np.uint16).ravel(), orc.F16, orc.I8, np.array([s_x32]), orc.SCALE_UNIFORM, M, K)
        qw = orc.quantize(w.view(np.uint16).ravel(), orc.F16, orc.I8, s_w32, orc.SCALE_ROW, N, K, N)
        xd = qx.astype(np.float64).reshape(M, K) * np.float64(s_x32)
        wd = qw.astype(np.float64).reshape(N, K) * s_w32.astype(np.float64)[:, None]
        core = xd @ wd.T
        bias = b.astype(np.float64)
        ref = core + bias
        # 1e-3 relative + one f16 rounding of the product + one of the sum with the bias
        tol = (1e-3 + 2.0 ** -10) * np.abs(core) + 2.0 ** -10 * np.abs(ref) + 1e-6
        assert np.all(np.abs(out - ref) <= tol), float(np.max(np.abs(out - ref) / (np.abs(ref) + 1e-9)))
        # a new weight tensor is picked up (the plan belongs to the parameter objects it was made from)
        lin.weight = tp.Tensor((2 * w.astype(np.float32)).astype(np.float16))
        lin.weight_scale = tp.Tensor((2 * s_w.astype(np.float32)).astype(np.float16))
        assert lin._prepared() is not plan
        out2 = lin(tp.Tensor(x)).torch().cpu().numpy().astype(np.float64)
        assert np.all(np.abs(out2 - (2 * core + bias)) <= 2 * tol)
        # an in-place update that torch cannot see is picked up after invalidate()
        plan2 = lin._prepared()
        lin.invalidate()
        assert lin._prepared() is not plan2
        # without the input scale there is no integer GEMM: the literal fake-quant form on the dense kernel
        lin.input_scale = None
        assert lin.route() == "dense"


@pytest.mark.parametrize("dname", ["float32", "bfloat16"])
def test_quant_linear_int8_keeps_the_module_dtype_outside_float16(tp, orc, pkg, dname):
    """A float32 or bfloat16 module with the same parameters stays on the literal form DQ(Q(x)) @ DQ(Q(W))^T in its own
    dtype: the W8A8 cluster writes f16, which would round every output to eleven bits and turn anything beyond 65504
    into inf.  Scales are chosen so that the outputs reach about 3e5."""
    import torch
    d = getattr(tp, dname)
    td = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dname]
    r = rng(79)
    M, K, N = 40, 256, 96
    x = torch.from_numpy((r.standard_normal((M, K)) * 30.0).astype(np.float32)).to(td)
    w = torch.from_numpy((r.standard_normal((N, K)) * 30.0).astype(np.float32)).to(td)
    w[:, :] = w.abs()                                  # no cancellation: every output is large
    x[:, :] = x.abs()
    s_x = (x.float().abs().max() / 127.0).to(td)
    s_w = (w.float().abs().amax(dim=1) / 127.0).to(td)
    lin = tp.Linear(K, N, bias=False, dtype=d, quant_dtype=tp.int8, weight_quant_dim=0)
    lin.load_state_dict({"weight": tp.Tensor(w, dtype=d), "weight_scale": tp.Tensor(s_w, dtype=d), "input_scale": tp.Tensor(s_x, dtype=d)})
    assert lin.route() == "dense"
    out = lin(tp.Tensor(x, dtype=d)).torch()
    assert pkg.last_kernel().startswith("mtrt_gemm_dense_")
    assert out.dtype == td and bool(torch.isfinite(out).all()) and float(out.float().max()) > 65504.0
    xq = torch.clamp(torch.round(x.float() / s_x.float()), -128, 127)
    wq = torch.clamp(torch.round(w.float() / s_w.float()[:, None]), -128, 127)
    xd = (xq * s_x.float()).to(td).double()           # the dequantized operands in the module's dtype
    wd = (wq * s_w.float()[:, None]).to(td).double()
    ref = xd @ wd.T
    ulp = {"float32": 2.0 ** -23, "bfloat16": 2.0 ** -7}[dname]
    assert bool(torch.all((out.cpu().double() - ref).abs() <= (ulp + 1e-5) * ref.abs()))


def test_quant_linear_int4_weight_only_runs_on_the_w4a16_cluster(tp, orc, pkg):
    """float16 module, int4 weight-only, per-output-channel scales: W4A16 cluster on a prepack made once; checked
    against the oracle's W4A16 program (same dequantize-then-accumulate order) and a float64 product."""
    import torch
    r = rng(78)
    M, K, N = 48, 256, 96
    x = r.standard_normal((M, K)).astype(np.float16)
    w = (r.standard_normal((N, K)) * 0.1).astype(np.float16)
    s_w = (np.abs(w.astype(np.float32)).max(axis=1) / 7.0).astype(np.float16)
    lin = tp.Linear(K, N, bias=False, dtype=tp.float16, quant_dtype=tp.int4, weight_quant_dim=0)
    lin.load_state_dict({"weight": tp.Tensor(w), "weight_scale": tp.Tensor(s_w)})
    assert lin.route() == "w4a16"
    out = lin(tp.Tensor(x)).torch()
    assert pkg.last_kernel().startswith("mtrt_gemm_w4a16_") and not pkg.last_kernel().endswith("_any")
    # oracle: codes [N,K] -> [K,N] packed, scales [1,N] with block = K
    codes = orc.quantize(w.view(np.uint16).ravel(), orc.F16, orc.I4, s_w.astype(np.float32), orc.SCALE_ROW, N, K, N)
    kn = np.ascontiguousarray(codes.reshape(N, K).T).ravel()
    packed = (kn[0::2] | (kn[1::2] << 4)).astype(np.uint8)
    ref = orc.gemm_w4a16(x.view(np.uint16), packed, s_w.view(np.uint16), K, N, K).ravel()
    got = out.view(torch.int16).cpu().numpy().view(np.uint16).ravel()
    gf, rf = orc.widen(got, orc.F16).astype(np.float64), orc.widen(ref, orc.F16).astype(np.float64)
    sgn = np.where(codes >= 8, codes.astype(np.int32) - 16, codes.astype(np.int32))
    wd = (sgn.reshape(N, K).astype(np.float32) * s_w.astype(np.float32)[:, None]).astype(np.float16).astype(np.float64)
    exact = x.astype(np.float64) @ wd.T
    mag = np.abs(x.astype(np.float64)) @ np.abs(wd.T)
    tol = 1e-3 * np.abs(exact) + 2.0 ** -10 * np.abs(exact) + 3e-6 * mag + 1e-7
    assert np.all(np.abs(gf - exact.ravel()) <= tol.ravel())
    assert np.all(np.abs(gf - rf) <= 2 * tol.ravel())
    # float32 module or a block-wise scale: dense route, same API
    lin32 = tp.Linear(K, N, bias=False, quant_dtype=tp.int4, weight_quant_dim=0)
    lin32.load_state_dict({"weight": tp.Tensor(w.astype(np.float32)), "weight_scale": tp.Tensor(s_w.astype(np.float32))})
    assert lin32.route() == "dense"
    o32 = lin32(tp.Tensor(x.astype(np.float32))).torch().cpu().numpy().astype(np.float64)
    assert pkg.last_kernel() == (("mtrt_gemm_dense_rows32_f32" if M <= 32 else "mtrt_gemm_dense_rows64_f32" if M <= 64 else "mtrt_gemm_dense_mfma_f32") if K % 32 == 0 else "mtrt_gemm_dense_edge_f32")
    wd32 = (sgn.reshape(N, K).astype(np.float32) * s_w.astype(np.float32)[:, None]).astype(np.float64)
    ex32 = x.astype(np.float64) @ wd32.T
    assert np.all(np.abs(o32 - ex32) <= 1e-5 * (np.abs(x.astype(np.float64)) @ np.abs(wd32.T)) + 1e-6)


@pytest.mark.parametrize("dname", ["float32", "float16", "bfloat16"])
def test_dense_linear_against_float64(tp, pkg, dname):
    """The unquantized module and ragged shapes on the dense kernel: f32 accumulation, result within the output
    type's rounding of the float64 product; leading batch dimensions are folded."""
    import torch
    d = getattr(tp, dname)
    td = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16}[dname]
    torch.manual_seed(5)
    for lead, K, N in (((3, 7), 50, 33), ((130,), 64, 129), ((1,), 1, 1), ((2, 300), 256, 520), ((700,), 1024, 8200), ((260,), 1031, 300), ((1,), 256, 40), ((2, 8), 4096, 1000), ((32,), 1024, 8209), ((5,), 64, 33), ((17,), 6144, 100), ((40,), 512, 300), ((64,), 128, 70), ((100,), 512, 300), ((2, 64), 256, 1000), ((65,), 2048, 33)):
        x = torch.randn(*lead, K, dtype=torch.float32).to(td)
        w = (torch.randn(N, K, dtype=torch.float32) * 0.2).to(td)
        b = torch.randn(N, dtype=torch.float32).to(td)
        lin = tp.Linear(K, N, dtype=d)
        lin.weight, lin.bias = tp.Tensor(w, dtype=d), tp.Tensor(b, dtype=d)
        out = lin(tp.Tensor(x, dtype=d)).torch()
        # operands whose rows are whole 128-byte slices of K run the 256 x 256 tile loop, everything else 128 x 128 tiles
        # with element-aligned loads; both on the matrix cores
        mfma = K % (32 if dname == "float32" else 64) == 0
        rows = int(np.prod(lead))                          # up to 128 rows read the weights once
        assert pkg.last_kernel() == ("mtrt_gemm_dense_rows32_" if mfma and rows <= 32 else "mtrt_gemm_dense_rows64_" if mfma and rows <= 64 else
                                     "mtrt_gemm_dense_rows128_" if mfma and rows <= 128 else
                                     "mtrt_gemm_dense_mfma_" if mfma else "mtrt_gemm_dense_edge_") + {"float32": "f32", "float16": "f16", "bfloat16": "bf16"}[dname]
        assert tuple(out.shape) == lead + (N,)
        ref = x.double() @ w.double().T + b.double()
        mag = x.double().abs() @ w.double().abs().T + b.double().abs()
        ulp = {"float32": 2.0 ** -23, "float16": 2.0 ** -10, "bfloat16": 2.0 ** -7}[dname]
        assert bool(torch.all((out.cpu().double() - ref).abs() <= ulp * ref.abs() + 1e-5 * mag + 1e-30))


def test_scale_from_amax(tp, orc):
    r = rng(5)
    x = r.standard_normal((64, 512)).astype(np.float32)
    amax, scale = tp.scale_from_amax(tp.Tensor(x), tp.float8)
    a_ref = orc.amax(x, orc.F32)
    assert np.float32(amax.item()).tobytes() == a_ref.tobytes()
    assert np.float32(scale.item()).tobytes() == orc.scale_from_amax(a_ref, 448.0).tobytes()


@pytest.mark.parametrize("normalized_shape", [(8, 4, 4), (4, 4)])
def test_layernorm_module_against_torch(tp, normalized_shape):
    """tripy/tests/integration/test_layernorm.py:57-109: unit weights give mean 0 / variance 1 over the
    normalized dimensions; with an affine transformation the result equals torch.nn.LayerNorm to atol 1e-6
    (f32) / 5e-3 (f16); eps = 0 and inputs U(0, 10) as there."""
    import torch
    torch.manual_seed(3)
    for d, atol in ((tp.float32, 1e-6), (tp.float16, 5e-3)):
        td = _torch_dtypes(tp)[d]
        ref = torch.nn.LayerNorm(normalized_shape=normalized_shape, eps=0.0, dtype=td, device="cuda")
        ln = tp.LayerNorm(normalized_shape=normalized_shape, eps=0.0, dtype=d)
        x = torch.empty(2, 8, 4, 4, dtype=td, device="cuda").uniform_(0, 10)
        ln.weight, ln.bias = tp.ones(normalized_shape, dtype=d), tp.zeros(normalized_shape, dtype=d)
        out = ln(tp.Tensor(x)).torch().float()
        dims = tuple(range(4 - len(normalized_shape), 4))
        assert out.mean(dim=dims).abs().mean().item() < 1e-4
        assert (out.var(dim=dims, unbiased=False) - 1).abs().mean().item() < (1e-4 if d == tp.float32 else 2e-3)
        torch.nn.init.uniform_(ref.weight, 0.2, 2)
        torch.nn.init.uniform_(ref.bias, 0.2, 2)
        ln.weight, ln.bias = tp.Tensor(ref.weight.to("cpu").detach()), tp.Tensor(ref.bias.to("cpu").detach())
        out = ln(tp.Tensor(x)).torch()
        with torch.no_grad():
            expected = ref(x)
        assert out.shape == expected.shape and out.dtype == expected.dtype
        assert torch.allclose(out, expected, atol=atol)


def test_layernorm_docstring_example(tp):
    """tripy/nvtripy/frontend/module/layernorm.py:116-133: iota weights and bias on a (2, 3) iota input."""
    import torch
    ln = tp.LayerNorm(3)
    ln.weight, ln.bias = tp.iota(ln.weight.shape), tp.iota(ln.bias.shape)
    x = tp.iota((2, 3), dim=1)
    out = ln(x)
    ref = torch.nn.LayerNorm(3)
    ref.weight.data, ref.bias.data = ln.weight.torch().cpu(), ln.bias.torch().cpu()
    assert out.shape == (2, 3)
    assert np.allclose(out.torch().cpu().numpy(), ref(x.torch().cpu()).detach().numpy())


@pytest.mark.parametrize("input_shape, dim", [((2, 2), 0), ((2,), 0), ((2, 2), None), ((2, 2), -1), ((3, 5, 7), 1), ((4,), -1)])
def test_softmax_against_torch(tp, input_shape, dim):
    """tripy/tests/integration/test_softmax.py:18-40 (atol 1e-4), plus a middle dimension and the rank-1
    input with dim = -1, which the reference sees as shape (n, 1): a softmax over one element."""
    import torch
    x = tp.iota(input_shape, dtype=tp.float32)
    out = tp.softmax(x, dim=dim)
    t = x.torch().cpu()
    if dim is None:
        expected = torch.softmax(t.flatten(), 0).reshape(input_shape)
    elif len(input_shape) == 1 and dim == -1:
        expected = torch.ones(input_shape)
    else:
        expected = torch.softmax(t, dim)
    assert out.shape == input_shape
    assert tp.allclose(out, tp.Tensor(expected), atol=1e-4)
