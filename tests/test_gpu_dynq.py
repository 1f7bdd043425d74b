"""Dynamic per-tensor quantization in one call (amax -> scale -> quantize -> dequantize): the one-launch kernel
against the CPU oracle and against the two launches it replaces, bit for bit; the bounded wait forced to give up
from the host; back-to-back launches on one stream (the scratch block restores itself)."""
import numpy as np
import pytest

from helpers import bits16, f32_bits, rng, to_device_float

pytestmark = pytest.mark.gpu

QMAX = {"i8": 127.0, "f8": 448.0}


def _types(pkg, orc, xname, qname):
    px, ox = {"f32": (pkg.F32, orc.F32), "f16": (pkg.F16, orc.F16), "bf16": (pkg.BF16, orc.BF16)}[xname]
    pq, oq = {"i8": (pkg.I8, orc.I8), "f8": (pkg.F8E4M3FN, orc.F8E4M3FN)}[qname]
    return px, ox, pq, oq


def _check(pkg, orc, x_f32, xname, qname, expect_kernel=None, flags=0, oflags=0):
    import torch
    px, ox, pq, oq = _types(pkg, orc, xname, qname)
    xd, xs = to_device_float(orc, x_f32, ox, "cuda:0")
    n = xs.size
    q, y, amax, scale = pkg.dynamic_quantize_dequantize(xd, pq, QMAX[qname], flags=flags)
    kernel = pkg.last_kernel()
    if expect_kernel:
        assert kernel == expect_kernel, kernel
    amax_ref = orc.amax(xs, ox)
    scale_ref = orc.scale_from_amax(amax_ref, QMAX[qname])
    assert f32_bits(amax.cpu().numpy())[0] == f32_bits(amax_ref)[0]
    assert f32_bits(scale.cpu().numpy())[0] == f32_bits(scale_ref)[0]
    q_ref = orc.quantize(xs, ox, oq, [scale_ref], orc.SCALE_UNIFORM, 1, n, 1, oflags)
    assert np.array_equal(q.cpu().numpy().view(np.uint8).ravel(), q_ref.view(np.uint8)), "codes (%s)" % kernel
    y_ref = orc.dequantize(q_ref, oq, ox, [scale_ref], orc.SCALE_UNIFORM, 1, n)
    got = y.cpu().numpy().ravel().view(np.uint32) if ox == orc.F32 else bits16(y)
    assert np.array_equal(got, y_ref.view(np.uint32) if ox == orc.F32 else y_ref), "dequantized values (%s)" % kernel
    return kernel


def test_c1_one_launch_full_size(pkg, orc):
    """BASELINE config 1 (f32 [1024, 4096] ~N(0,1), seed 1, int8, amax / 127) in one launch, and the same bits
    from the two launches it replaces."""
    import torch
    x = rng(1).standard_normal((1024, 4096), dtype=np.float32)
    orc.set_threads(16)
    assert _check(pkg, orc, x, "f32", "i8", "mtrt_dynqdq_f32_i8_v4") == "mtrt_dynqdq_f32_i8_v4"
    orc.set_threads(1)
    xd = torch.from_numpy(x).cuda()
    q1, y1, a1, s1 = pkg.dynamic_quantize_dequantize(xd, pkg.I8, 127.0)
    a2, s2 = pkg.amax(xd, 127.0)
    q2, y2 = pkg.quantize_dequantize(xd, s2.reshape(1), pkg.I8)
    assert torch.equal(q1, q2) and torch.equal(y1.view(torch.int32), y2.view(torch.int32))
    assert torch.equal(torch.stack([a1, s1]).view(torch.int32), torch.stack([a2, s2]).view(torch.int32))


@pytest.mark.parametrize("xname", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("qname", ["i8", "f8"])
def test_type_pairs_and_grid_sizes(pkg, orc, xname, qname):
    g = rng(hash((xname, qname)) % 1000)
    k = "mtrt_dynqdq_%s_%s_" % (xname, qname)
    grp = 4 if xname == "f32" else 8
    # one workgroup (partly filled), a few workgroups with a ragged last one, and the 16-vector form
    for n, kernel in ((grp * 37, k + "v4"), (grp * (1024 * 4 * 3 + 555), k + "v4"), (grp * 1024 * 4 * 256 + grp * 1024 * 16 * 3, k + "v16")):
        x = (g.standard_normal(n) * 3).astype(np.float32)
        orc.set_threads(16)
        if kernel.endswith("v16") and grp == 8 and qname == "f8":
            # no 16-vector form for the 16-bit -> f8 pairs (it would need scratch memory): the two launches
            assert _check(pkg, orc, x, xname, qname).startswith("mtrt_qdq_")
        else:
            _check(pkg, orc, x, xname, qname, kernel)
        orc.set_threads(1)


def test_flags_zero_tensor_and_two_launch_route(pkg, orc):
    import torch
    g = rng(9)
    x = (g.standard_normal(4096 * 8) * 50).astype(np.float32)
    _check(pkg, orc, x, "bf16", "f8", "mtrt_dynqdq_bf16_f8_v4", flags=pkg.Q_ROUND_TO_INT, oflags=orc.Q_ROUND_TO_INT)
    _check(pkg, orc, x, "f32", "f8", "mtrt_dynqdq_f32_f8_v4", flags=pkg.F8_VIA_F16, oflags=orc.F8_VIA_F16)
    # n not a multiple of the vector length: reduction + element-wise pass, same results
    k = _check(pkg, orc, x[:4099], "f32", "i8")
    assert k.startswith("mtrt_qdq_"), k
    # all zeros: scale 0, every quotient 0 / 0
    xd = torch.zeros(8192, device="cuda")
    q1, y1, a1, s1 = pkg.dynamic_quantize_dequantize(xd, pkg.I8, 127.0)
    assert pkg.last_kernel() == "mtrt_dynqdq_f32_i8_v4"
    a2, s2 = pkg.amax(xd, 127.0)
    q2, y2 = pkg.quantize_dequantize(xd, s2.reshape(1), pkg.I8)
    assert torch.equal(q1, q2) and torch.equal(y1.view(torch.int32), y2.view(torch.int32)) and s1.item() == 0.0
    # codes only
    q3, y3, _, _ = pkg.dynamic_quantize_dequantize(torch.from_numpy(x).cuda(), pkg.I8, 127.0, dequantize=False)
    assert y3 is None
    s = orc.scale_from_amax(orc.amax(x, orc.F32), 127.0)
    assert np.array_equal(q3.cpu().numpy(), orc.quantize(x, orc.F32, orc.I8, [s], orc.SCALE_UNIFORM, 1, x.size))
    L = pkg.lib()
    st = torch.cuda.current_stream().cuda_stream
    assert L.mtrt_hip_dynamic_quantize_dequantize(st, xd.data_ptr(), pkg.F32, q1.data_ptr(), pkg.I4, None, 8192, 7.0, None,
                                                  a1.data_ptr(), 0) == 1
    assert L.mtrt_hip_dynamic_quantize_dequantize(st, xd.data_ptr(), pkg.F32, q1.data_ptr(), pkg.I8, None, 8192, 127.0, None,
                                                  None, 0) == 1
    assert b"scale_out" in L.mtrt_hip_last_error()


def test_bounded_wait_gives_up_cleanly_and_block_restores_itself(pkg, orc):
    """With the poll budget at zero no workgroup waits for the grid's maximum: each one that did not arrive last
    reduces the whole tensor itself.  Same bits; and the stream's reduction block is back to zero afterwards, which
    the following ordinary launches (amax and the one-launch form, several in a row) depend on."""
    import torch
    L = pkg.lib()
    x = rng(2).standard_normal(1024 * 4 * 4 * 40 + 4 * 100, dtype=np.float32)
    old = L.mtrt_hip_set_wait_limit(0)
    try:
        orc.set_threads(16)
        _check(pkg, orc, x, "f32", "i8", "mtrt_dynqdq_f32_i8_v4")
        _check(pkg, orc, x * 0.5, "bf16", "f8", "mtrt_dynqdq_bf16_f8_v4")
    finally:
        assert L.mtrt_hip_set_wait_limit(old) == 0
        orc.set_threads(1)
    xd = torch.from_numpy(x).cuda()
    for scale in (1.0, 3.0, 0.25):
        xs = (xd * scale).contiguous()
        a, s = pkg.amax(xs, 127.0)
        q1, y1, a1, s1 = pkg.dynamic_quantize_dequantize(xs, pkg.I8, 127.0)
        assert torch.equal(torch.stack([a, s]).view(torch.int32), torch.stack([a1, s1]).view(torch.int32))
        q2, y2 = pkg.quantize_dequantize(xs, s.reshape(1), pkg.I8)
        assert torch.equal(q1, q2) and torch.equal(y1.view(torch.int32), y2.view(torch.int32))
