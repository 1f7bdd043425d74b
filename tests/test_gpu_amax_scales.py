"""Per-channel / block-wise amax + scale (mtrt_hip_amax_scales) against the CPU oracle, bit for bit: the per-token
activation scales of BASELINE config 4 and the [K / 128, N] int4 block scales of config 5 at full size, every
addressing on ragged and unaligned shapes, and the whole calibration -> quantize chain."""
import numpy as np
import pytest

from helpers import f32_bits, rng, to_device_float

pytestmark = pytest.mark.gpu


def _run(pkg, orc, x_f32, xname, kind_name, d0, d1, nb, qmax, expect_kernel=None):
    px, ox = {"f32": (pkg.F32, orc.F32), "f16": (pkg.F16, orc.F16), "bf16": (pkg.BF16, orc.BF16)}[xname]
    pk, ok = {"row": (pkg.SCALE_ROW, orc.SCALE_ROW), "col": (pkg.SCALE_COL, orc.SCALE_COL),
              "uniform": (pkg.SCALE_UNIFORM, orc.SCALE_UNIFORM)}[kind_name]
    xd, xs = to_device_float(orc, x_f32.reshape(d0, d1), ox, "cuda:0")
    amax, scale = pkg.amax_scales(xd, qmax, pk, d0, d1, nb)
    if expect_kernel:
        assert pkg.last_kernel() == expect_kernel, pkg.last_kernel()
    a_ref, s_ref = orc.amax_scales(xs, ox, ok, d0, d1, nb, qmax)
    assert np.array_equal(f32_bits(amax.cpu().numpy()), f32_bits(a_ref)), "amax (%s)" % pkg.last_kernel()
    assert np.array_equal(f32_bits(scale.cpu().numpy()), f32_bits(s_ref)), "scale (%s)" % pkg.last_kernel()
    return xd, scale, s_ref, xs


def test_c4_per_token_activation_scales(pkg, orc):
    """Config 4: activations [2048, 4096]; a_scale[m] = max_k |a[m, k]| / 127, then the int8 codes of the GEMM."""
    M, K = 2048, 4096
    a = (rng(4).standard_normal((M, K)) * 3).astype(np.float32)
    orc.set_threads(16)
    xd, scale, s_ref, xs = _run(pkg, orc, a, "f16", "row", M, K, M, 127.0, "mtrt_amax_rows_f16")
    q = pkg.quantize(xd, scale, pkg.I8, pkg.SCALE_ROW, M, K, M)
    q_ref = orc.quantize(xs, orc.F16, orc.I8, s_ref, orc.SCALE_ROW, M, K, M)
    orc.set_threads(1)
    assert np.array_equal(q.cpu().numpy().ravel(), q_ref)
    assert int(np.abs(q_ref.astype(np.int32)).reshape(M, K).max(axis=1).min()) == 127      # every row uses the full range


def test_c5_int4_block_scales(pkg, orc):
    """Config 5: weights [4096, 11008], blocks of 128 rows: scale [32, 11008] = block amax / 7, then the int4 codes."""
    K, N, B = 4096, 11008, 128
    w = (rng(5).standard_normal((K, N)) * 0.05).astype(np.float32)
    orc.set_threads(16)
    xd, scale, s_ref, xs = _run(pkg, orc, w, "f16", "col", K, N, B, 7.0, "mtrt_amax_cols_f16")
    q = pkg.quantize(xd, scale, pkg.I4_PACKED, pkg.SCALE_COL, K, N, B)
    q_ref = orc.quantize(xs, orc.F16, orc.I4_PACKED, s_ref, orc.SCALE_COL, K, N, B)
    orc.set_threads(1)
    assert np.array_equal(q.cpu().numpy().ravel(), q_ref)


@pytest.mark.parametrize("xname", ["f32", "f16", "bf16"])
def test_every_addressing_on_ragged_shapes(pkg, orc, xname):
    g = rng(17)
    grp = 4 if xname == "f32" else 8
    k = "_" + xname
    cases = [
        ("row", 37, 16 * grp * 9 + grp, 37, "mtrt_amax_rows" + k),          # one scale per row (one tile each: no sharing)
        ("row", 60, grp * 5, 12, "mtrt_amax_finish" + k),                    # channel on a middle axis: 5 rows per scale, two workgroups each
        ("row", 9, 131, 9, "mtrt_amax_rows_any" + k),                        # row length not a vector multiple
        ("row", 1, 7, 1, "mtrt_amax_rows_any" + k),
        ("col", 48, grp * 70, 16, "mtrt_amax_cols" + k),                     # two strips of 64 vectors, 16-row blocks
        ("col", 40, grp * 3, 40, "mtrt_amax_cols" + k),                      # per channel on the last axis
        ("col", 6, grp * 2, 1, "mtrt_amax_cols" + k),                        # block of one row: amax = |x|
        ("col", 30, 77, 5, "mtrt_amax_cols_u" + k),                         # row length not a vector multiple: vectors at element alignment
        ("col", 8, grp * 70 + 3, 4, "mtrt_amax_cols_u" + k),                  # two strips and a partial last vector
        ("col", 260, grp * 2 + 1, 130, "mtrt_amax_finish" + k),               # long ragged blocks: rows dealt to several workgroups
        ("uniform", 11, 100, 1, "mtrt_amax" + k),
    ]
    for kind, d0, d1, nb, kernel in cases:
        x = (g.standard_normal(d0 * d1) * 4).astype(np.float32)
        _run(pkg, orc, x, xname, kind, d0, d1, nb, 448.0, kernel)


@pytest.mark.parametrize("xname", ["f32", "f16", "bf16"])
def test_per_channel_scales_of_a_k_by_n_weight(pkg, orc, xname):
    """Few, long column blocks (per-output-channel scales of a [K, N] weight, nb = K): the rows of a block are dealt
    to several workgroups that meet by atomic max, then a finishing launch writes amax and scale.  Full-size config-4
    weight, a block length that is not a multiple of the part length, two blocks, and only one of the two outputs."""
    import torch
    grp = 4 if xname == "f32" else 8
    g = rng(23)
    orc.set_threads(16)
    try:
        cases = [(4096, 11008, 4096), (1000, grp * 33, 1000), (512, grp * 70, 256), (130, grp * 3, 130)]
        for d0, d1, nb in cases:
            x = (g.standard_normal(d0 * d1) * 0.3).astype(np.float32)
            x[g.integers(0, x.size, 50)] *= 40.0
            xd, scale, s_ref, xs = _run(pkg, orc, x, xname, "col", d0, d1, nb, 127.0, "mtrt_amax_finish_" + xname)
        # the scales alone (amax_out NULL), then the amax alone: the words the workgroups meet in are the output's own
        px = {"f32": pkg.F32, "f16": pkg.F16, "bf16": pkg.BF16}[xname]
        L = pkg.lib()
        st = torch.cuda.current_stream().cuda_stream
        only = torch.full((d1,), 7.0, dtype=torch.float32, device="cuda")
        pkg.check(L.mtrt_hip_amax_scales(st, xd.data_ptr(), px, pkg.SCALE_COL, d0, d1, nb, 127.0, None, only.data_ptr()))
        assert np.array_equal(f32_bits(only.cpu().numpy()), f32_bits(s_ref))
        pkg.check(L.mtrt_hip_amax_scales(st, xd.data_ptr(), px, pkg.SCALE_COL, d0, d1, nb, 127.0, only.data_ptr(), None))
        a_ref, _ = orc.amax_scales(xs, {"f32": orc.F32, "f16": orc.F16, "bf16": orc.BF16}[xname], orc.SCALE_COL, d0, d1, nb, 127.0)
        assert np.array_equal(f32_bits(only.cpu().numpy()), f32_bits(a_ref))
    finally:
        orc.set_threads(1)


@pytest.mark.parametrize("xname", ["f32", "f16", "bf16"])
def test_few_row_scales_share_workgroups(pkg, orc, xname):
    """Row kind with a handful of scales (a short channel axis in front of large inner extents, or a few very long
    rows): several workgroups per scale meet by atomic max, then the finishing launch.  Rows per scale that differ
    (37 rows, 5 scales), rows longer than one tile of 1024 vectors, one scale."""
    grp = 4 if xname == "f32" else 8
    g = rng(31)
    orc.set_threads(16)
    try:
        for d0, d1, nb in ((512, grp * 300, 8), (8, grp * 5000, 8), (37, grp * 130, 5), (2048, grp * 64, 64), (3, grp * 2049, 1)):
            x = (g.standard_normal(d0 * d1) * 0.7).astype(np.float32)
            x[g.integers(0, x.size, 20)] *= 30.0
            _run(pkg, orc, x, xname, "row", d0, d1, nb, 127.0, "mtrt_amax_finish_" + xname)
    finally:
        orc.set_threads(1)


def test_argument_checks_and_empty(pkg):
    import torch
    L = pkg.lib()
    x = torch.zeros(64, device="cuda")
    out = torch.zeros(64, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    call = lambda kind, d0, d1, nb: L.mtrt_hip_amax_scales(s, x.data_ptr(), pkg.F32, kind, d0, d1, nb, 127.0, None, out.data_ptr())
    assert call(pkg.SCALE_COL, 8, 8, 3) == 1 and b"does not divide" in L.mtrt_hip_last_error()
    assert call(pkg.SCALE_ROW, 8, 8, 9) == 1
    assert call(pkg.SCALE_ROW, 8, 8, 0) == 1
    assert call(5, 8, 8, 1) == 1
    assert call(pkg.SCALE_ROW, 0, 8, 4) == 0 and call(pkg.SCALE_COL, 8, 0, 4) == 0
    assert L.mtrt_hip_amax_scales(s, x.data_ptr(), pkg.F32, pkg.SCALE_ROW, 8, 8, 8, 127.0, None, None) == 1
