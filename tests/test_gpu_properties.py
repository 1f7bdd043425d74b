"""Size-independent properties at the full sizes of BASELINE.json's configurations, checked on the GPU without the
oracle: what must hold whatever the inputs are (idempotence of quantize after dequantize, a maximum of maxima, rows
that do not know about each other, softmax rows that sum to one), so that the kernels' indexing at full size (tile maps,
chunking, tails) is covered by a second, independent kind of evidence beside the bit-exact comparisons with the oracle."""
import numpy as np
import pytest

from helpers import rng

pytestmark = pytest.mark.gpu


def _c3_tensor(torch):
    g = torch.Generator(device="cuda")
    g.manual_seed(3)
    x = torch.randn((16384, 8192), generator=g, device="cuda") * (2.0 ** 0.5)
    x[torch.rand((16384, 8192), generator=g, device="cuda") < 0.001] *= 50.0
    return x.to(torch.bfloat16)


def test_requantizing_the_dequantized_tensor_gives_the_same_codes(pkg):
    """Q(DQ(Q(x))) = Q(x) and DQ of it the same values, for C1 (f32 -> int8) and C3 (bf16 -> f8E4M3FN) at full size:
    a dequantized value is its code times the scale, rounded once, and divides back to within half a code step."""
    import torch
    x1 = torch.from_numpy(rng(1).standard_normal((1024, 4096), dtype=np.float32)).cuda()
    for x, qd, qmax in ((x1, pkg.I8, 127.0), (_c3_tensor(torch), pkg.F8E4M3FN, 448.0)):
        _, scale = pkg.amax(x, qmax)
        q, y = pkg.quantize_dequantize(x, scale.reshape(1), qd)
        q2, y2 = pkg.quantize_dequantize(y, scale.reshape(1), qd)
        assert torch.equal(q.view(torch.uint8), q2.view(torch.uint8)), pkg.last_kernel()
        assert torch.equal(y.view(torch.int16 if y.dtype == torch.bfloat16 else torch.int32),
                           y2.view(torch.int16 if y.dtype == torch.bfloat16 else torch.int32))
        # and the separate launches agree with the fused one
        q3 = pkg.quantize(x, scale.reshape(1), qd)
        assert torch.equal(q.view(torch.uint8), q3.view(torch.uint8))


def test_amax_is_the_maximum_of_the_amax_of_its_parts(pkg):
    """C3 at full size: the reduction over the whole tensor equals the maximum over reductions of uneven pieces (a
    checksum of checksums), is blind to the sign, and the scale is amax / 448 in one IEEE division."""
    import torch
    x = _c3_tensor(torch)
    amax, scale = pkg.amax(x, 448.0)
    flat = x.view(-1)
    cuts = [0, 1, 4097, 10 ** 6 + 3, 2 ** 26 - 8, 2 ** 26 + 5, flat.numel()]
    parts = [pkg.amax(flat[a:b].contiguous(), 448.0)[0] for a, b in zip(cuts[:-1], cuts[1:])]
    assert float(torch.stack(parts).max()) == float(amax)
    assert float(pkg.amax((-x).contiguous(), 448.0)[0]) == float(amax)
    assert float(amax) == float(x.float().abs().max())
    assert np.float32(float(scale)) == np.float32(float(amax)) / np.float32(448.0)


def test_softmax_and_layernorm_rows_at_full_size(pkg):
    """C2b: every one of the 4096 x 4096 softmax rows is non-negative, sums to one within the f16 rounding of 4096
    terms, and keeps the order of its inputs.  C2a: every LayerNorm row with gamma = 1, beta = 0 has mean 0 and
    variance 1 within the bf16 rounding of its outputs.  A row's result does not depend on the rows around it."""
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(22)
    x = (torch.randn((4096, 4096), generator=g, device="cuda") * 2.0).half()
    y = pkg.softmax(x)
    s = y.float().sum(dim=1)
    assert float(y.min()) >= 0.0
    assert float((s - 1.0).abs().max()) <= 4096 * 2.0 ** -12 * float(y.float().max())
    assert float((s - 1.0).abs().max()) <= 2e-3
    order_in = x[::257].float().argsort(dim=1, stable=True)
    ys = torch.gather(y[::257].float(), 1, order_in)
    assert bool((ys[:, 1:] >= ys[:, :-1]).all())          # a larger input never gets a smaller output
    rows = torch.tensor([0, 1, 63, 64, 2047, 4095], device="cuda")
    assert torch.equal(pkg.softmax(x[rows].contiguous()).view(torch.int16), y[rows].view(torch.int16))

    xb = (torch.randn((8192, 4096), generator=g, device="cuda") * 3.0 + 0.5).bfloat16()
    gamma = torch.ones(4096, device="cuda", dtype=torch.bfloat16)
    beta = torch.zeros(4096, device="cuda", dtype=torch.bfloat16)
    z = pkg.layernorm(xb, gamma, beta, 1e-5).float()
    assert float(z.mean(dim=1).abs().max()) <= 2e-3
    assert float((z.var(dim=1, unbiased=False) - 1.0).abs().max()) <= 5e-3
    rows = torch.tensor([0, 5, 4096, 8191], device="cuda")
    z2 = pkg.layernorm(xb[rows].contiguous(), gamma, beta, 1e-5)
    assert torch.equal(z2.float(), z[rows])


def test_gemm_rows_do_not_know_about_each_other(pkg):
    """C4 (W8A8, M = 2048) and C5 (W4A16, M = 4096) at full size: permuting the rows of the activations permutes the rows
    of the result and changes no bit (every output row is summed in the same order wherever its tile lies), and the
    first 300 rows computed on their own (other kernels: other tiles, other tile maps) give the same bits for the
    integer GEMM."""
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(45)
    M, K, N = 2048, 4096, 11008
    a = torch.clamp(torch.round(torch.randn((M, K), generator=g, device="cuda") * 40), -128, 127).to(torch.int8)
    w = torch.clamp(torch.round(torch.randn((K, N), generator=g, device="cuda") * 40), -128, 127).to(torch.int8)
    a_s = torch.rand(M, generator=g, device="cuda") * 0.015 + 0.005
    w_s = torch.rand(N, generator=g, device="cuda") * 0.015 + 0.005
    wf = pkg.gemm_w8a8_prepack_fragments(w)
    y = pkg.gemm_w8a8_fragments(a, wf, a_s, w_s, N)
    print("C4 kernel:", pkg.last_kernel(), flush=True)
    perm = torch.randperm(M, generator=g, device="cuda")
    yp = pkg.gemm_w8a8_fragments(a[perm].contiguous(), wf, a_s[perm].contiguous(), w_s, N)
    assert torch.equal(yp.view(torch.int16), y[perm].view(torch.int16))
    ys = pkg.gemm_w8a8_fragments(a[:300].contiguous(), wf, a_s[:300].contiguous(), w_s, N)
    assert torch.equal(ys.view(torch.int16), y[:300].view(torch.int16)), pkg.last_kernel()
    del a, w, wf, y, yp

    M, B = 4096, 128
    a = torch.randn((M, K), generator=g, device="cuda").half()
    wq = torch.randint(0, 256, (K * N // 2,), generator=g, device="cuda", dtype=torch.uint8)
    s = (torch.rand((K // B, N), generator=g, device="cuda") * 0.015 + 0.005).half()
    wp = pkg.gemm_w4a16_prepack(wq, K, N)
    y = pkg.gemm_w4a16(a, s, K, N, B, w_prepacked=wp)
    print("C5 kernel:", pkg.last_kernel(), flush=True)
    perm = torch.randperm(M, generator=g, device="cuda")
    yp = pkg.gemm_w4a16(a[perm].contiguous(), s, K, N, B, w_prepacked=wp)
    assert torch.equal(yp.view(torch.int16), y[perm].view(torch.int16))
