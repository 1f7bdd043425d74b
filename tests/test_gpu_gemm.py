"""Parity of the GEMM clusters with the CPU oracle, through the C ABI.

W8A8: the int32 accumulators are exact under any summation order and the epilogue is a
fixed chain of correctly rounded f32 operations followed by one f16 narrowing, so the
f16 outputs must be BIT-IDENTICAL to the oracle's.
"""
import numpy as np
import pytest

from helpers import bits16, rng

pytestmark = pytest.mark.gpu


def _w8a8_inputs(g, M, K, N):
    a = np.clip(np.rint(g.standard_normal((M, K)) * 40), -128, 127).astype(np.int8)
    w = np.clip(np.rint(g.standard_normal((K, N)) * 40), -128, 127).astype(np.int8)
    a_s = g.uniform(0.005, 0.02, M).astype(np.float32)
    w_s = g.uniform(0.005, 0.02, N).astype(np.float32)
    return a, w, a_s, w_s


def _run_w8a8(pkg, a, w, a_s, w_s):
    import torch
    ad, wd = torch.from_numpy(a).cuda(), torch.from_numpy(w).cuda()
    w_nk = pkg.gemm_w8a8_prepack(wd)
    assert torch.equal(w_nk, wd.t().contiguous())
    y = pkg.gemm_w8a8(ad, w_nk, torch.from_numpy(a_s).cuda(), torch.from_numpy(w_s).cuda())
    return y, pkg.last_kernel()


@pytest.mark.parametrize("shape", [(256, 128, 128), (512, 512, 256), (300, 256, 200), (1, 128, 1), (37, 384, 129),
                                   (257, 1024, 130)])
def test_w8a8_mfma_kernel_small_shapes(pkg, orc, shape):
    M, K, N = shape
    a, w, a_s, w_s = _w8a8_inputs(rng(M + K + N), M, K, N)
    y, kernel = _run_w8a8(pkg, a, w, a_s, w_s)
    assert kernel == "mtrt_gemm_w8a8_nk"
    assert np.array_equal(bits16(y).reshape(M, N), orc.gemm_w8a8(a, w, a_s, w_s))


@pytest.mark.parametrize("shape", [(5, 7, 3), (33, 100, 65), (2, 130, 4)])
def test_w8a8_generic_kernel(pkg, orc, shape):
    M, K, N = shape
    a, w, a_s, w_s = _w8a8_inputs(rng(M * K + N), M, K, N)
    y, kernel = _run_w8a8(pkg, a, w, a_s, w_s)
    assert kernel == "mtrt_gemm_w8a8_nk_any"
    assert np.array_equal(bits16(y).reshape(M, N), orc.gemm_w8a8(a, w, a_s, w_s))


def test_w8a8_extreme_values_do_not_overflow(pkg, orc):
    M, K, N = 64, 4096, 128
    a = np.full((M, K), -128, np.int8)
    w = np.full((K, N), -128, np.int8)
    w[:, ::2] = 127
    a_s = np.full(M, 2.0 ** -12, np.float32)
    w_s = np.full(N, 2.0 ** -12, np.float32)
    y, _ = _run_w8a8(pkg, a, w, a_s, w_s)
    assert np.array_equal(bits16(y).reshape(M, N), orc.gemm_w8a8(a, w, a_s, w_s))
    got = y.float().cpu().numpy()
    assert got[0, 1] == 4096 * 128 * 128 / 2.0 ** 24 and got[0, 0] == -4096 * 128 * 127 / 2.0 ** 24


def test_c4_w8a8_full_size(pkg, orc):
    """BASELINE config 4: M=2048 K=4096 N=11008, values clip(rint(N(0,40))), seed 4.  The oracle
    evaluates one whole 256-row tile (every lane/accumulator position of the kernel) plus rows
    from every other tile; all N columns of those rows are compared bit for bit."""
    import torch
    M, K, N = 2048, 4096, 11008
    a, w, a_s, w_s = _w8a8_inputs(rng(4), M, K, N)
    y, kernel = _run_w8a8(pkg, a, w, a_s, w_s)
    assert kernel == "mtrt_gemm_w8a8_nk"
    got = bits16(y).reshape(M, N)
    orc.set_threads(16)
    ref = orc.gemm_w8a8(a, w, a_s, w_s, m0=768, mcount=256)
    assert np.array_equal(got[768:1024], ref)
    for m0 in (0, 255, 256, 600, 1100, 1500, 1800, 2047):
        assert np.array_equal(got[m0:m0 + 1], orc.gemm_w8a8(a, w, a_s, w_s, m0=m0, mcount=1))
    orc.set_threads(1)
    # independent whole-matrix check: float64 GEMM of the same integers on the GPU, same epilogue
    acc = (torch.from_numpy(a).cuda().double() @ torch.from_numpy(w).cuda().double())
    expect = ((acc.float() * torch.from_numpy(a_s).cuda()[:, None]) * torch.from_numpy(w_s).cuda()[None, :]).half()
    assert torch.equal(y, expect)


def test_w8a8_argument_checks(pkg):
    import torch
    L = pkg.lib()
    t = torch.zeros(256, device="cuda")
    assert L.mtrt_hip_gemm_w8a8(None, t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), -1, 128, 4) == 1
    assert L.mtrt_hip_gemm_w8a8(None, None, t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), 4, 128, 4) == 1
    assert L.mtrt_hip_gemm_w8a8(None, t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), 0, 128, 4) == 0
