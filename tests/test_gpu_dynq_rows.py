"""Dynamic per-row (per-token) quantization in one call: amax per row -> scale = amax / qmax -> quantize, against the
CPU oracle (the composition of its pinned per-row amax / scale and row-scaled quantize) and against the two launches
the call is defined by, bit for bit: the wave-per-row and workgroup-per-row forms, every type pair, ragged shapes that
fall back to the two launches, rows of zeros, flags, argument checks."""
import numpy as np
import pytest

from helpers import f32_bits, rng, to_device_float

pytestmark = pytest.mark.gpu

QMAX = {"i8": 127.0, "f8": 448.0}


def _types(pkg, orc, xname, qname):
    px, ox = {"f32": (pkg.F32, orc.F32), "f16": (pkg.F16, orc.F16), "bf16": (pkg.BF16, orc.BF16)}[xname]
    pq, oq = {"i8": (pkg.I8, orc.I8), "f8": (pkg.F8E4M3FN, orc.F8E4M3FN)}[qname]
    return px, ox, pq, oq


def _check(pkg, orc, x_f32, xname, qname, expect=None, flags=0, oflags=0, omode=None):
    """x_f32: [rows, d].  Returns the kernel of the last launch."""
    import torch
    px, ox, pq, oq = _types(pkg, orc, xname, qname)
    rows, d = x_f32.shape
    xd, xs = to_device_float(orc, x_f32, ox, "cuda:0")
    print("case: dynamic_quantize_rows", x_f32.shape, xname, qname, "flags", flags, flush=True)
    q, amax, scale = pkg.dynamic_quantize_rows(xd, pq, QMAX[qname], flags=flags)
    kernel = pkg.last_kernel()
    if expect:
        assert kernel == expect, kernel
    amax_ref, scale_ref = orc.amax_scales(xs, ox, orc.SCALE_ROW, rows, d, rows, QMAX[qname])
    assert np.array_equal(f32_bits(amax.cpu().numpy()), f32_bits(amax_ref)), "amax (%s)" % kernel
    assert np.array_equal(f32_bits(scale.cpu().numpy()), f32_bits(scale_ref)), "scale (%s)" % kernel
    q_ref = orc.quantize(xs, ox, oq, scale_ref, orc.SCALE_ROW, rows, d, rows, oflags, orc.IEEE if omode is None else omode)
    assert np.array_equal(q.cpu().numpy().view(np.uint8).ravel(), q_ref.view(np.uint8)), "codes (%s)" % kernel
    # the two launches the call is defined by
    a2, s2 = pkg.amax_scales(xd, QMAX[qname], pkg.SCALE_ROW, rows, d, rows)
    q2 = pkg.quantize(xd, s2, pq, pkg.SCALE_ROW, rows, d, rows, flags)
    assert torch.equal(q.view(torch.uint8), q2.view(torch.uint8))
    assert torch.equal(torch.stack([amax, scale]).view(torch.int32), torch.stack([a2, s2]).view(torch.int32))
    return kernel


def test_c4_activations_full_size(pkg, orc):
    """The activations of BASELINE config 4 before quantization: f16 [2048, 4096], per-token int8 codes and scales."""
    x = (rng(4).standard_normal((2048, 4096), dtype=np.float32) * 3.0)
    orc.set_threads(16)
    # (few enough rows that the four waves of a workgroup share each one)
    assert _check(pkg, orc, x, "f16", "i8") in ("mtrt_dynq_rows_f16_i8_g4v2", "mtrt_dynq_rows_f16_i8_v8")
    orc.set_threads(1)


@pytest.mark.parametrize("xname", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("qname", ["i8", "f8"])
def test_type_pairs_and_row_lengths(pkg, orc, xname, qname):
    """One vector per row up to the longest row a wave holds, then the workgroup form up to its longest; row counts
    that leave the last workgroup of the wave form partly filled."""
    import torch
    g = rng(sum(map(ord, xname + qname)))
    grp = 4 if xname == "f32" else 8
    many = 16 * torch.cuda.get_device_properties(0).multi_processor_count + 3   # more rows than the workgroup form is used for
    k = "mtrt_dynq_rows_%s_%s_" % (xname, qname)
    orc.set_threads(16)
    for rows, nvec, kernel in ((1, 1, "v1"), (5, 37, "v1"), (7, 64, "v1"), (6, 65, "v2"), (9, 200, "v4"), (3, 512, "g4v2"),
                               (4, 256, "g4v1"), (10, 1000, "g4v4"), (2, 1024, "g4v4"), (3, 1025, "g4v8"), (5, 300 * 4 + 7, "g4v8"),
                               (2, 4096, "g4v16"), (131, 96, "v2"), (many, 264, "v8"), (many + 1, 136, "v4")):
        x = (g.standard_normal((rows, nvec * grp)) * g.uniform(0.1, 30.0, (rows, 1))).astype(np.float32)
        if kernel == "g4v16" and grp == 8 and qname == "f8":
            # the 16-vector form of the 16-bit -> f8 pairs is not built (it would need scratch memory): two launches
            assert _check(pkg, orc, x, xname, qname).startswith("mtrt_q_row")
            continue
        _check(pkg, orc, x, xname, qname, k + kernel)
    orc.set_threads(1)


def test_rows_that_take_the_two_launches(pkg, orc):
    """Rows that are not whole vectors, rows longer than a workgroup holds, and an operand off 16-byte alignment: the
    same results through the reduction and the row-scaled quantize pass."""
    import torch
    g = rng(12)
    orc.set_threads(16)
    for shape, xname in (((33, 1001), "f32"), ((4, 70001), "f16"), ((3, 32768 + 8), "bf16"), ((2, 16384 + 4), "f32")):
        x = (g.standard_normal(shape) * 5).astype(np.float32)
        k = _check(pkg, orc, x, xname, "i8")
        assert k.startswith("mtrt_q_row"), k
    orc.set_threads(1)
    # x one element off 16-byte alignment
    buf = torch.randn(8 * 256 + 1, device="cuda")
    xd = buf[1:].view(8, 256)
    q, amax, scale = pkg.dynamic_quantize_rows(xd, pkg.I8, 127.0)
    assert pkg.last_kernel().startswith("mtrt_q_row")
    xs = xd.cpu().numpy()
    a_ref, s_ref = orc.amax_scales(xs.ravel(), orc.F32, orc.SCALE_ROW, 8, 256, 8, 127.0)
    assert np.array_equal(f32_bits(scale.cpu().numpy()), f32_bits(s_ref))
    assert np.array_equal(q.cpu().numpy(), orc.quantize(xs.ravel(), orc.F32, orc.I8, s_ref, orc.SCALE_ROW, 8, 256, 8))


def test_zero_rows_flags_and_special_values(pkg, orc):
    """A row of zeros has scale 0 and every quotient 0 / 0; rows with an infinity; the f8 flags."""
    g = rng(13)
    x = (g.standard_normal((12, 768)) * 2).astype(np.float32)
    x[3] = 0.0
    x[5, 17] = np.inf
    x[7, :] = -0.0
    x[9, 100] = 1e-40          # a subnormal among ordinary values
    x[10] = 1e-41              # a row of subnormals: a scale below the range of the short division
    _check(pkg, orc, x, "f32", "i8", "mtrt_dynq_rows_f32_i8_v4")
    _check(pkg, orc, x, "f32", "f8", "mtrt_dynq_rows_f32_f8_v4")
    y = (g.standard_normal((12, 768)) * 40).astype(np.float32)
    _check(pkg, orc, y, "bf16", "f8", "mtrt_dynq_rows_bf16_f8_v2", flags=pkg.Q_ROUND_TO_INT, oflags=orc.Q_ROUND_TO_INT)
    _check(pkg, orc, y, "f32", "f8", "mtrt_dynq_rows_f32_f8_v4", flags=pkg.F8_VIA_F16, oflags=orc.F8_VIA_F16)
    _check(pkg, orc, y, "f16", "f8", "mtrt_dynq_rows_f16_f8_v2", flags=pkg.F8_REFHOST, omode=orc.REFHOST)


def test_feeds_the_w8a8_gemm(pkg, orc):
    """Per-token codes and scales from this call are what the W8A8 GEMM takes as a and a_scale."""
    import torch
    g = rng(14)
    M, K, N = 96, 512, 160
    x = torch.from_numpy((g.standard_normal((M, K)) * 2).astype(np.float16)).cuda()
    w = np.clip(np.rint(g.standard_normal((K, N)) * 40), -128, 127).astype(np.int8)
    w_s = g.uniform(0.005, 0.02, N).astype(np.float32)
    q, _, a_s = pkg.dynamic_quantize_rows(x, pkg.I8, 127.0, want_amax=False)
    wf = pkg.gemm_w8a8_prepack_fragments(torch.from_numpy(w).cuda())
    y = pkg.gemm_w8a8_fragments(q.view(M, K), wf, a_s, torch.from_numpy(w_s).cuda(), N)
    ref = orc.gemm_w8a8(q.cpu().numpy().reshape(M, K), w, a_s.cpu().numpy(), w_s)
    assert np.array_equal(y.view(torch.int16).cpu().numpy().view(np.uint16), ref.reshape(M, N))


def test_argument_checks(pkg):
    import torch
    L = pkg.lib()
    st = torch.cuda.current_stream().cuda_stream
    x = torch.zeros(64, device="cuda")
    q = torch.zeros(64, dtype=torch.int8, device="cuda")
    s = torch.zeros(8, device="cuda")
    call = L.mtrt_hip_dynamic_quantize_rows
    assert call(st, x.data_ptr(), pkg.F32, q.data_ptr(), pkg.I4, 8, 8, 7.0, None, s.data_ptr(), 0) == 1
    assert call(st, x.data_ptr(), pkg.F32, q.data_ptr(), pkg.I8, 8, 8, 127.0, None, None, 0) == 1
    assert b"scale_out" in L.mtrt_hip_last_error()
    assert call(st, x.data_ptr(), pkg.F32, q.data_ptr(), pkg.I8, -1, 8, 127.0, None, s.data_ptr(), 0) == 1
    assert call(st, None, pkg.F32, q.data_ptr(), pkg.I8, 8, 8, 127.0, None, s.data_ptr(), 0) == 1
    assert call(st, x.data_ptr(), pkg.F32, q.data_ptr(), pkg.F8E4M3FN, 8, 8, 448.0, None, s.data_ptr(), 6) == 1
    assert call(st, x.data_ptr(), pkg.F32, q.data_ptr(), pkg.I8, 0, 8, 127.0, None, s.data_ptr(), 0) == 0
    assert call(st, x.data_ptr(), pkg.F32, q.data_ptr(), pkg.I8, 8, 0, 127.0, None, s.data_ptr(), 0) == 0
