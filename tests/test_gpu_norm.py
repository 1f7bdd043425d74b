"""Parity of the fused LayerNorm and softmax clusters with the CPU oracle.

These are floating-point programs whose reductions the GPU evaluates as trees and
the host evaluates left to right, so results are compared under a stated tolerance:

  * against the float64 evaluation of the same formula:
        |got - exact| <= 1e-3 * |exact| + 0.5 ulp_out(exact) + 2e-5 * cond
    (1e-3 relative is the bar for fp16/bf16 outputs; the half ulp is the rounding every
    implementation, the oracle included, must commit when it stores the narrow type;
    `cond` is the magnitude of the terms whose f32 rounding errors the result inherits:
    |d*rstd*gamma| + |beta| for LayerNorm, where the two can cancel to a result far
    smaller than either, and 0 for softmax, which has no cancellation);
  * against the oracle's stored output: at most 1 ulp of the output type (+ the same
    cond term) apart on every element, and bit-identical on all but a small fraction
    (a 1e-6 relative difference before the store flips the rounding of about
    1e-6/2^-9 of bf16 values).  f32 outputs: 2e-5 relative to |exact| + cond.
"""
import numpy as np
import pytest

from helpers import float_storage, rng, to_device_float

pytestmark = pytest.mark.gpu

ULP_REL = {"f32": 2.0 ** -23, "f16": 2.0 ** -10, "bf16": 2.0 ** -7}
MIN_NORMAL = {"f32": 2.0 ** -126, "f16": 2.0 ** -14, "bf16": 2.0 ** -126}


def _x(pkg, orc, name):
    return {"f32": (pkg.F32, orc.F32), "f16": (pkg.F16, orc.F16), "bf16": (pkg.BF16, orc.BF16)}[name]


def _ulp(v, name):
    """Spacing of the output type at magnitude |v| (subnormal spacing below the least normal)."""
    a = np.maximum(np.abs(v), MIN_NORMAL[name])
    return 2.0 ** np.floor(np.log2(a)) * ULP_REL[name]


def _compare(orc, name, got_store, ref_store, exact, max_mismatch_frac, cond=None, oracle_slack=1.0):
    o = {"f32": orc.F32, "f16": orc.F16, "bf16": orc.BF16}[name]
    got = orc.widen(got_store, o).astype(np.float64) if o != orc.F32 else got_store.astype(np.float64)
    ref = orc.widen(ref_store, o).astype(np.float64) if o != orc.F32 else ref_store.astype(np.float64)
    exact = exact.ravel()
    slack = 2e-5 * (np.zeros_like(exact) if cond is None else cond.ravel())
    err = np.abs(got - exact)
    if name == "f32":
        bound = 2e-5 * np.abs(exact) + slack + 1e-37
        assert np.all(err <= bound), "vs float64: max excess %r" % (err - bound).max()
        # oracle_slack > 1: rows so long that the host's left-to-right f32 sums are themselves outside the bound
        # (65536 terms: the oracle is 2.7 bounds from the float64 value; the tree sums on the GPU stay inside one)
        assert np.all(np.abs(got - ref) <= 2 * bound * oracle_slack)
        return 0.0
    ulp = _ulp(exact, name)
    bound = 1e-3 * np.abs(exact) + 0.5 * ulp * 1.0001 + slack + 1e-45
    worst = np.argmax(err - bound)
    assert np.all(err <= bound), "vs float64: element %d got %r exact %r" % (worst, got[worst], exact[worst])
    d = np.abs(got - ref)
    assert np.all(d <= _ulp(ref, name) * 1.0001 + 2 * slack), "more than 1 ulp from the oracle: max %r" % d.max()
    frac = np.count_nonzero(got_store != ref_store) / got_store.size
    assert frac <= max_mismatch_frac, "fraction of elements not bit-identical to the oracle: %g" % frac
    return frac


def _layernorm_f64(x, g, b, eps):
    mu = x.mean(axis=1, keepdims=True)
    d = x - mu
    var = (d * d).mean(axis=1, keepdims=True)
    t = d / np.sqrt(var + eps) * g
    return t + b, np.abs(t) + np.abs(b)


def _softmax_f64(x):
    e = np.exp(x - x.max(axis=1, keepdims=True))
    return e / e.sum(axis=1, keepdims=True)


def _run_layernorm(pkg, orc, name, rows, d, seed, expect_kernel=None, frac=2e-3, oracle_slack=1.0):
    p, o = _x(pkg, orc, name)
    g = rng(seed)
    x = g.standard_normal((rows, d), dtype=np.float32)
    gamma = g.uniform(0.5, 1.5, d).astype(np.float32)
    beta = (g.standard_normal(d, dtype=np.float32) * np.float32(0.1))
    xd, xs = to_device_float(orc, x, o, "cuda:0")
    gd, gs = to_device_float(orc, gamma, o, "cuda:0")
    bd, bs = to_device_float(orc, beta, o, "cuda:0")
    y = pkg.layernorm(xd, gd, bd, 1e-5)
    if expect_kernel:
        assert pkg.last_kernel() == expect_kernel
    y_ref = orc.layernorm(xs, gs, bs, o, rows, d, 1e-5)
    w = (lambda a: orc.widen(a, o).astype(np.float64)) if o != orc.F32 else (lambda a: a.astype(np.float64))
    exact, cond = _layernorm_f64(w(xs).reshape(rows, d), w(gs), w(bs), 1e-5)
    return _compare(orc, name, float_storage(orc, y, o), y_ref, exact, frac, cond, oracle_slack)


def _run_softmax(pkg, orc, name, rows, d, seed, expect_kernel=None, frac=2e-3, sigma=2.0):
    p, o = _x(pkg, orc, name)
    x = rng(seed).standard_normal((rows, d), dtype=np.float32) * np.float32(sigma)
    xd, xs = to_device_float(orc, x, o, "cuda:0")
    y = pkg.softmax(xd)
    if expect_kernel:
        assert pkg.last_kernel() == expect_kernel
    y_ref = orc.softmax(xs, o, rows, d)
    w = (lambda a: orc.widen(a, o).astype(np.float64)) if o != orc.F32 else (lambda a: a.astype(np.float64))
    exact = _softmax_f64(w(xs).reshape(rows, d))
    got = float_storage(orc, y, o)
    fr = _compare(orc, name, got, y_ref, exact, frac)
    gotf = w(got).reshape(rows, d)
    assert np.all(np.abs(gotf.sum(axis=1) - 1.0) < 2e-3 if name != "f32" else np.abs(gotf.sum(axis=1) - 1.0) < 1e-5)
    return fr


def test_c2a_layernorm_bf16_full_size(pkg, orc):
    """BASELINE config 2a: bf16 [8192,4096], x~N(0,1), gamma~U(0.5,1.5), beta~N(0,0.1), eps 1e-5, seed 2."""
    orc.set_threads(16)
    _run_layernorm(pkg, orc, "bf16", 8192, 4096, 2, "mtrt_layernorm_bf16_v8" + ("r" if _resident(8192) else ""))
    orc.set_threads(1)


def test_c2b_softmax_f16_full_size(pkg, orc):
    """BASELINE config 2b: f16 [4096,4096], logits ~N(0,4) read as variance 4 (sigma 2), seed 2."""
    orc.set_threads(16)
    _run_softmax(pkg, orc, "f16", 4096, 4096, 2, "mtrt_softmax_f16_v8")
    orc.set_threads(1)


@pytest.mark.parametrize("name", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", [(5, 8), (33, 512), (7, 1000), (3, 4104), (2, 8192), (9, 16384), (4, 331), (1, 1), (6, 40000)])
def test_layernorm_shapes(pkg, orc, name, shape):
    # Long rows: the host's left-to-right f32 sums drift from the tree sums by a few 1e-6
    # relative, which moves proportionally more stored values across a rounding boundary.
    frac = 2e-3 if shape[1] <= 8192 else 2e-2
    _run_layernorm(pkg, orc, name, shape[0], shape[1], 20 + shape[1] % 97, frac=frac)


@pytest.mark.parametrize("name", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", [(5, 8), (33, 512), (7, 1000), (3, 4104), (2, 8192), (9, 16384), (4, 331), (1, 1), (6, 40000)])
def test_softmax_shapes(pkg, orc, name, shape):
    # what differs from the host is mostly the order of the row sum; the share of stored values it moves across a
    # rounding boundary grows with the row length.
    frac = 2e-3 if shape[1] <= 8192 else 2e-2
    _run_softmax(pkg, orc, name, shape[0], shape[1], 40 + shape[1] % 97, frac=frac)


def _resident(rows):
    """The dispatch rule of the eight-vector LayerNorm: the 64-register kernel when eight waves per SIMD hold
    every row at once and five would not."""
    import torch
    simds = 4 * torch.cuda.get_device_properties(0).multi_processor_count
    return 5 * simds < rows <= 8 * simds


def test_layernorm_resident_variant_window_and_bits(pkg, orc):
    """Both eight-vector kernels run the same arithmetic: rows just inside the window (64-register kernel)
    give the bits of the same rows launched below it (default kernel); the window's edges pick the kernels."""
    import torch
    simds = 4 * torch.cuda.get_device_properties(0).multi_processor_count
    d = 4096
    torch.manual_seed(5)
    g = (torch.rand(d, device="cuda") + 0.5).to(torch.bfloat16)
    b = (torch.randn(d, device="cuda") * 0.1).to(torch.bfloat16)
    x = torch.randn(8 * simds + 1, d, device="cuda").to(torch.bfloat16)
    lo = pkg.layernorm(x[:5 * simds], g, b, 1e-5)
    assert pkg.last_kernel() == "mtrt_layernorm_bf16_v8"
    mid = pkg.layernorm(x[:5 * simds + 1], g, b, 1e-5)
    assert pkg.last_kernel() == "mtrt_layernorm_bf16_v8r"
    top = pkg.layernorm(x[:8 * simds], g, b, 1e-5)
    assert pkg.last_kernel() == "mtrt_layernorm_bf16_v8r"
    over = pkg.layernorm(x, g, b, 1e-5)
    assert pkg.last_kernel() == "mtrt_layernorm_bf16_v8"
    assert torch.equal(lo.view(torch.int16), mid[:5 * simds].view(torch.int16))
    assert torch.equal(top.view(torch.int16), over[:8 * simds].view(torch.int16))
    assert torch.equal(lo.view(torch.int16), over[:5 * simds].view(torch.int16))
    # a ragged row length (not all 64 * 8 vectors used) through the 64-register kernel
    d2 = 4000
    x2 = torch.randn(5 * simds + 7, d2, device="cuda").to(torch.float16)
    g2 = (torch.rand(d2, device="cuda") + 0.5).half()
    b2 = (torch.randn(d2, device="cuda") * 0.1).half()
    a = pkg.layernorm(x2, g2, b2, 1e-5)
    assert pkg.last_kernel() == "mtrt_layernorm_f16_v8r"
    c = pkg.layernorm(x2[:100], g2, b2, 1e-5)
    assert pkg.last_kernel() == "mtrt_layernorm_f16_v8"
    assert torch.equal(a[:100].view(torch.int16), c.view(torch.int16))


def test_kernel_selection(pkg, orc):
    import torch
    for d, k in ((512, "v1"), (1024, "v2"), (2048, "v4"), (4096, "v8"), (8192, "v16"), (8200, "g256v8"), (131080, "any"), (331, "u64v1"), (5, "u8v1"), (1, "u8v1")):
        x = torch.randn(4, d, device="cuda", dtype=torch.bfloat16)
        pkg.softmax(x)
        assert pkg.last_kernel() == "mtrt_softmax_bf16_" + k
        pkg.layernorm(x, torch.ones(d, device="cuda", dtype=torch.bfloat16), torch.zeros(d, device="cuda", dtype=torch.bfloat16), 1e-5)
        assert pkg.last_kernel() == "mtrt_layernorm_bf16_" + k
    # a row pointer that is not 16-byte aligned takes the kernels that move vectors at element alignment
    buf = torch.randn(4 * 512 + 1, device="cuda", dtype=torch.bfloat16)
    got = pkg.softmax(buf[1:].view(4, 512))
    assert pkg.last_kernel() == "mtrt_softmax_bf16_u64v1"
    want = pkg.softmax(buf[1:].view(4, 512).clone())
    assert pkg.last_kernel() == "mtrt_softmax_bf16_v1"
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_softmax_extremes_and_empty(pkg, orc):
    import torch
    # widely spread logits: the largest entry dominates, tiny ones underflow to 0 or f16 subnormals
    _run_softmax(pkg, orc, "f16", 16, 4096, 5, sigma=8.0)
    _run_softmax(pkg, orc, "f32", 16, 1024, 6, sigma=30.0)
    x = torch.full((3, 256), -7.0, device="cuda", dtype=torch.float32)
    y = pkg.softmax(x)
    assert torch.equal(y, torch.full_like(y, 1.0 / 256))
    assert pkg.softmax(torch.empty((0, 64), device="cuda")).numel() == 0
    z = torch.zeros((2, 128), device="cuda", dtype=torch.bfloat16)
    out = pkg.layernorm(z, torch.ones(128, device="cuda", dtype=torch.bfloat16),
                        torch.full((128,), 0.5, device="cuda", dtype=torch.bfloat16), 1e-5)
    assert torch.equal(out, torch.full_like(out, 0.5))


def test_more_rows_than_the_row_per_wave_grid_covers(pkg, orc):
    """The one-wave-per-row kernels do not loop over rows and their grid is capped at 2^20 workgroups of four
    rows; beyond 2^22 rows the looping kernels must take over so that the last rows are still written."""
    import torch
    rows, d = (1 << 22) + 7, 8
    x = torch.randn(rows, d, device="cuda", dtype=torch.float16)
    y = torch.full_like(x, float("nan"))
    pkg.softmax(x, out=y)
    assert pkg.last_kernel() == "mtrt_softmax_f16_any"
    torch.cuda.synchronize()
    assert bool(torch.isfinite(y).all())
    tail = slice(rows - 64, rows)
    xs = bits16_of(x[tail])
    ref = orc.softmax(xs, orc.F16, 64, d)
    got = bits16_of(y[tail])
    assert np.max(np.abs(orc.widen(got, orc.F16) - orc.widen(ref, orc.F16))) <= 2.0 ** -10
    g = torch.ones(d, device="cuda", dtype=torch.float16)
    b = torch.zeros(d, device="cuda", dtype=torch.float16)
    z = torch.full_like(x, float("nan"))
    pkg.layernorm(x, g, b, 1e-5, out=z)
    assert pkg.last_kernel() == "mtrt_layernorm_f16_any"
    torch.cuda.synchronize()
    assert bool(torch.isfinite(z).all())
    refz = orc.layernorm(xs, bits16_of(g), bits16_of(b), orc.F16, 64, d, 1e-5)
    gotz = bits16_of(z[tail])
    assert np.max(np.abs(orc.widen(gotz, orc.F16) - orc.widen(refz, orc.F16))) <= 2.0 ** -8


def bits16_of(t):
    from helpers import bits16
    return bits16(t)


def _group_cases(name):
    """(row length, kernel suffix) across the limits of the workgroup-per-row kernels: 256 or 1024 lanes with 8 or 16
    vectors each, rows that fill them exactly and rows that do not, and the first length beyond them."""
    e = 4 if name == "f32" else 8
    return [(e * 1025, "_g256v8"), (e * 2048, "_g256v8"), (e * 2049, "_g256v16"), (e * 4096, "_g256v16"),
            (e * 4097, "_g1024v8"), (e * 8192, "_g1024v8"), (e * 8193, "_g1024v16"), (e * 16032, "_g1024v16"),
            (e * 16384, "_g1024v16"), (e * 16385, "_any")]


@pytest.mark.parametrize("name", ["f32", "f16", "bf16"])
def test_layernorm_rows_owned_by_a_workgroup(pkg, orc, name):
    """Hidden sizes beyond one wave's registers (1024 vectors): one workgroup per row, the row still read once."""
    for d, suffix in _group_cases(name):
        # beyond 40000 elements the host's running sums drift further from the tree sums: up to 5 % of the stored
        # 16-bit values then sit on the other side of a rounding boundary (all within one ulp, all inside the float64 bound)
        _run_layernorm(pkg, orc, name, 3, d, 60 + d % 89, "mtrt_layernorm_" + name + suffix, frac=2e-2 if d <= 40000 else 5e-2,
                       oracle_slack=4.0 if d > 40000 else 1.0)


@pytest.mark.parametrize("name", ["f32", "f16", "bf16"])
def test_softmax_rows_owned_by_a_workgroup(pkg, orc, name):
    """Vocabulary-sized rows (e.g. 128256 = 8 * 16032 logits): one workgroup per row."""
    for d, suffix in _group_cases(name):
        _run_softmax(pkg, orc, name, 3, d, 70 + d % 89, "mtrt_softmax_" + name + suffix, frac=2e-2 if d <= 40000 else 5e-2)


def _ragged_cases(name, layernorm=False):
    """(row length, kernel suffix): lengths that are not whole vectors (attention rows of 77, 197, 1500 keys; a
    50257-entry vocabulary) in every scheme, from one vector plus one element up to 1024 x 16 vectors plus a tail;
    rows of at most 32 vectors share a wave (8, 16 or 32 lanes each) whether or not they are whole vectors."""
    e = 4 if name == "f32" else 8
    cases = _ragged_cases_by_length(e)
    if name == "f32" and layernorm:
        # the eight-vector f32 LayerNorm kernels at element alignment compile to 230 registers: the host takes the
        # sixteen-vector forms for those rows
        cases = [(d, s.replace("v8", "v16")) for d, s in cases]
    return cases


def _ragged_cases_by_length(e):
    return [(1, "_u8v1"), (2, "_u8v1"), (e - 1, "_u8v1"), (e + 1, "_u8v1"), (77, "_u16v1" if e == 8 else "_u32v1"), (197, "_u32v1" if e == 8 else "_u64v1"), (e * 8, "_u8v1"),
            (e * 32, "_u32v1"), (e * 32 + 1, "_u32v1"), (e * 33 + 1, "_u64v1"), (e * 64 + 3, "_u64v1"), (e * 65 + 3, "_u64v2"), (1500 if e == 8 else 1501, "_u64v4" if e == 8 else "_u64v8"),
            (e * 512 + e - 1, "_u64v8"), (e * 1024 + 1, "_u64v16"), (e * 1025 + 2, "_u256v8"), (e * 4096 + 3, "_u256v16"),
            (50257, "_u1024v8" if e == 8 else "_u1024v16"), (e * 16384 + e - 1, "_u1024v16"), (e * 16385 + 1, "_any")]


@pytest.mark.parametrize("name", ["f32", "f16", "bf16"])
def test_layernorm_ragged_rows(pkg, orc, name):
    for d, suffix in _ragged_cases(name, layernorm=True):
        _run_layernorm(pkg, orc, name, 5, d, 80 + d % 89, "mtrt_layernorm_" + name + suffix, frac=2e-2 if d <= 40000 else 5e-2,
                       oracle_slack=4.0 if d > 40000 else 1.0)


@pytest.mark.parametrize("name", ["f32", "f16", "bf16"])
def test_softmax_ragged_rows(pkg, orc, name):
    for d, suffix in _ragged_cases(name):
        _run_softmax(pkg, orc, name, 5, d, 90 + d % 89, "mtrt_softmax_" + name + suffix, frac=2e-2 if d <= 40000 else 5e-2)
