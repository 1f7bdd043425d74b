"""Pins the program-level functions of the CPU oracle (oracle/programs.cpp) without a GPU,
by checks that do not retype the oracle's own loops:
  - numpy / torch library routines that the programs reduce to (rint, clip, float32 divide,
    float16 casts, int64 matmul, torch layer_norm / softmax in float64);
  - scale-indexing invariants built so that a wrong index (row/col swapped, interleaved instead of
    contiguous blocks, wrong nibble) changes the answer;
  - the value-level known answers of the reference's Tripy / JAX / StableHLO tests.
"""
import numpy as np
import pytest

from helpers import rng


def test_amax_and_scale(orc):
    x = rng(1).standard_normal(10007, dtype=np.float32)
    x[123] = -9.75
    assert orc.amax(x, orc.F32) == np.float32(9.75)
    assert orc.scale_from_amax(np.float32(9.75), 127.0) == np.float32(9.75) / np.float32(127.0)
    xb = orc.narrow(x, orc.BF16)
    assert orc.amax(xb, orc.BF16) == np.abs(orc.widen(xb, orc.BF16)).max()
    assert orc.amax(np.zeros(0, dtype=np.float32), orc.F32) == 0.0


def test_amax_per_scale_element_closed_form(orc):
    """Per-channel and block-wise amax against numpy's reductions over the reshaped tensor; the scale is one f32
    divide per element.  The index invariants tell the addressings apart: per-row vs per-channel-of-a-middle-axis
    (rows r and r + C share), blocks of rows per column vs per-column over all rows."""
    g = rng(11)
    x = (g.standard_normal((24, 40)) * 5).astype(np.float32)
    ax = np.abs(x)
    a, s = orc.amax_scales(x, orc.F32, orc.SCALE_ROW, 24, 40, 24, 127.0)           # one scale per row
    assert np.array_equal(a, ax.max(axis=1)) and np.array_equal(s, (ax.max(axis=1) / np.float32(127.0)).astype(np.float32))
    a, _ = orc.amax_scales(x, orc.F32, orc.SCALE_ROW, 24, 40, 6, 127.0)            # [4, 6, 40], channel axis 1
    assert np.array_equal(a, ax.reshape(4, 6, 40).max(axis=(0, 2)))
    a, s = orc.amax_scales(x, orc.F32, orc.SCALE_COL, 24, 40, 8, 7.0)              # blocks of 8 rows per column
    assert np.array_equal(a, ax.reshape(3, 8, 40).max(axis=1).ravel())
    assert np.array_equal(s, (ax.reshape(3, 8, 40).max(axis=1).ravel() / np.float32(7.0)).astype(np.float32))
    a, _ = orc.amax_scales(x, orc.F32, orc.SCALE_COL, 24, 40, 24, 448.0)           # per channel on the last axis
    assert np.array_equal(a, ax.max(axis=0))
    a, s = orc.amax_scales(x, orc.F32, orc.SCALE_UNIFORM, 24, 40, 1, 448.0)
    assert a[0] == ax.max() and s[0] == np.float32(ax.max()) / np.float32(448.0)
    xb = orc.narrow(x, orc.BF16)
    a, _ = orc.amax_scales(xb, orc.BF16, orc.SCALE_COL, 24, 40, 8, 7.0)
    assert np.array_equal(a, np.abs(orc.widen(xb, orc.BF16)).reshape(3, 8, 40).max(axis=1).ravel())
    # quantizing with those scales uses the whole code range and never saturates past it
    a, s = orc.amax_scales(x, orc.F32, orc.SCALE_COL, 24, 40, 8, 7.0)
    q = orc.quantize(x, orc.F32, orc.I4, s, orc.SCALE_COL, 24, 40, 8)
    codes = np.where(q >= 8, q.astype(np.int32) - 16, q.astype(np.int32)).reshape(3, 8, 40)
    assert np.array_equal(np.abs(codes).max(axis=1).ravel(), np.full(120, 7))


@pytest.mark.parametrize("qd,lo,hi", [("I8", -128, 127), ("I4", -8, 7)])
def test_quantize_int_closed_form(orc, qd, lo, hi):
    g = rng(2)
    d0, d1 = 24, 40
    x = (g.standard_normal((d0, d1)) * 30).astype(np.float32)
    q_dt = getattr(orc, qd)
    # per-tensor
    s = np.float32(0.37)
    expect = np.clip(np.rint(x / s), lo, hi).astype(np.int8)
    got = orc.quantize(x, orc.F32, q_dt, [s], orc.SCALE_UNIFORM, d0, d1)
    assert np.array_equal(orc.widen(got, q_dt).astype(np.int8), expect.ravel())
    # per-channel on axis 0 (row scales) and on the last axis (column scales)
    sr = g.uniform(0.1, 2.0, d0).astype(np.float32)
    got = orc.quantize(x, orc.F32, q_dt, sr, orc.SCALE_ROW, d0, d1, d0)
    assert np.array_equal(orc.widen(got, q_dt).astype(np.int8), np.clip(np.rint(x / sr[:, None]), lo, hi).astype(np.int8).ravel())
    sc = g.uniform(0.1, 2.0, d1).astype(np.float32)
    got = orc.quantize(x, orc.F32, q_dt, sc, orc.SCALE_COL, d0, d1, d0)
    assert np.array_equal(orc.widen(got, q_dt).astype(np.int8), np.clip(np.rint(x / sc[None, :]), lo, hi).astype(np.int8).ravel())
    # contiguous blocks of 8 rows along axis 0: scale[r // 8, c]   (TensorRTOps.td:3120-3121, 3417-3436)
    sb = g.uniform(0.1, 2.0, (d0 // 8, d1)).astype(np.float32)
    got = orc.quantize(x, orc.F32, q_dt, sb.ravel(), orc.SCALE_COL, d0, d1, 8)
    expect = np.clip(np.rint(x / np.repeat(sb, 8, axis=0)), lo, hi).astype(np.int8)
    assert np.array_equal(orc.widen(got, q_dt).astype(np.int8), expect.ravel())
    interleaved = np.clip(np.rint(x / np.tile(sb, (8, 1))), lo, hi).astype(np.int8)
    assert not np.array_equal(expect, interleaved)          # the check can tell the two layouts apart
    # blocks of 10 along the last axis: scale[r, c // 10]
    sl = g.uniform(0.1, 2.0, (d0, d1 // 10)).astype(np.float32)
    got = orc.quantize(x, orc.F32, q_dt, sl.ravel(), orc.SCALE_ROW, d0 * (d1 // 10), 10, d0 * (d1 // 10))
    expect = np.clip(np.rint(x / np.repeat(sl, 10, axis=1)), lo, hi).astype(np.int8)
    assert np.array_equal(orc.widen(got, q_dt).astype(np.int8), expect.ravel())
    # middle axis of a rank-3 tensor [3, 8, 40]: d0 = 24 rows, scale[row % 8]
    sm = g.uniform(0.1, 2.0, 8).astype(np.float32)
    got = orc.quantize(x, orc.F32, q_dt, sm, orc.SCALE_ROW, d0, d1, 8)
    expect = np.clip(np.rint(x.reshape(3, 8, d1) / sm[None, :, None]), lo, hi).astype(np.int8)
    assert np.array_equal(orc.widen(got, q_dt).astype(np.int8), expect.ravel())


def test_quantize_packed_int4_nibble_order(orc):
    x = np.float32([[0, 1, 2, 3], [-1, -2, -8, 7]])
    got = orc.quantize(x, orc.F32, orc.I4_PACKED, [np.float32(1)], orc.SCALE_UNIFORM, 2, 4)
    assert list(got) == [0x10, 0x32, 0xEF, 0x78]             # element 2i in the low nibble
    assert np.array_equal(orc.unpack_int4(got, 8), x.ravel().astype(np.int8))
    un = orc.quantize(x, orc.F32, orc.I4, [np.float32(1)], orc.SCALE_UNIFORM, 2, 4)
    assert list(un) == [0, 1, 2, 3, 0xF, 0xE, 0x8, 0x7]      # one per byte, low nibble, upper nibble clear


def test_quantize_packed_rows_of_odd_length_with_threads(orc):
    """Rows of odd length share bytes with their neighbours: the threaded run must equal the nibbles of the
    one-code-per-byte form (two rows of one element each, the case two threads would split)."""
    g = rng(61)
    orc.set_threads(8)
    try:
        for _ in range(1500):
            x = (g.standard_normal((2, 1)) * 3).astype(np.float32)
            one_per_byte = orc.quantize(x, orc.F32, orc.I4, [np.float32(1)], orc.SCALE_UNIFORM, 2, 1)
            packed = orc.quantize(x, orc.F32, orc.I4_PACKED, [np.float32(1)], orc.SCALE_UNIFORM, 2, 1)
            assert packed[0] == (one_per_byte[0] | (one_per_byte[1] << 4))
    finally:
        orc.set_threads(1)


def test_quantize_fp8_forms(orc):
    import torch
    g = rng(3)
    x = (g.standard_normal(4096) * 100).astype(np.float32)
    s = np.float32(0.61)
    v = np.clip(x / s, -448, 448).astype(np.float32)
    expect = torch.from_numpy(v).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = orc.quantize(x, orc.F32, orc.F8E4M3FN, [s], orc.SCALE_UNIFORM, 1, x.size)
    assert np.array_equal(got, expect)
    vr = np.clip(np.rint(x / s), -448, 448).astype(np.float32)
    expect_r = torch.from_numpy(vr).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got_r = orc.quantize(x, orc.F32, orc.F8E4M3FN, [s], orc.SCALE_UNIFORM, 1, x.size, 1, orc.Q_ROUND_TO_INT)
    assert np.array_equal(got_r, expect_r) and not np.array_equal(got, got_r)
    # StableHLO fixture raise-qdq-per-tensor-quantize.mlir:82-95: bf16 [1, 2] / 0.5 -> f8 [2, 4]
    xb = orc.narrow(np.float32([1.0, 2.0]), orc.BF16)
    q = orc.quantize(xb, orc.BF16, orc.F8E4M3FN, [np.float32(0.5)], orc.SCALE_UNIFORM, 1, 2, 1, orc.Q_ROUND_TO_INT)
    assert list(orc.widen(q, orc.F8E4M3FN)) == [2.0, 4.0]
    # refhost mode: exponent-15 results collapse to 448
    big = np.float32([250, 300, 440, -260])
    q = orc.quantize(big, orc.F32, orc.F8E4M3FN, [np.float32(1)], orc.SCALE_UNIFORM, 1, 4, 1, 0, orc.REFHOST)
    assert list(orc.widen(q, orc.F8E4M3FN)) == [448.0, 448.0, 448.0, -448.0]


def test_quantize_fp8_via_f16_double_rounding(orc):
    """The reference's GPU code generator converts f32 -> f16 -> f8 (NormalizeQuantizedConversions.cpp:38-118), two
    roundings to nearest even.  Pinned as a composition of two independently pinned steps: numpy's float16 cast,
    then the f16 -> f8 table minted from the reference's compiled DataTypes.cpp (IEEE-agreeing entries only:
    |v| < 248 and outside the subnormal-carry window, where the host class is correct RNE)."""
    import os
    one = [np.float32(1)]
    # hand-derived witnesses: 1.0625 is the midpoint of the f8 neighbours 1.0 (0x38, even) and 1.125 (0x39).
    # 1.0625 + 2^-20 lies above it (direct: 0x39) but rounds to 1.0625 in f16 (ulp 2^-10), a tie -> even -> 0x38.
    # 1.1875 is the midpoint of 1.125 (0x39, odd) and 1.25 (0x3A): from below, direct gives 0x39, via f16 0x3A.
    w = np.float32([1.0625 + 2.0 ** -20, -(1.0625 + 2.0 ** -20), 1.1875 - 2.0 ** -20, 1.0625, 1.0625 + 2.0 ** -10])
    direct = orc.quantize(w, orc.F32, orc.F8E4M3FN, one, orc.SCALE_UNIFORM, 1, w.size)
    via = orc.quantize(w, orc.F32, orc.F8E4M3FN, one, orc.SCALE_UNIFORM, 1, w.size, 1, orc.F8_VIA_F16)
    assert list(direct) == [0x39, 0xB9, 0x39, 0x38, 0x39]
    assert list(via) == [0x38, 0xB8, 0x3A, 0x38, 0x39]
    # composition against numpy + the golden table, on normally distributed quotients
    tab = np.load(os.path.join(os.path.dirname(__file__), "golden", "lowp_from_f16_grid.npz"))
    f16_to_f8_ref = tab["f8"]                      # reference host class applied to every f16 value (index = f16 bits)
    x = (rng(31).standard_normal(1 << 18) * 60).astype(np.float32)
    x = x[(np.abs(x) < 240) & (np.abs(x) > 0.02)]  # where the host class equals IEEE (quirks Q1-Q3 excluded)
    via = orc.quantize(x, orc.F32, orc.F8E4M3FN, one, orc.SCALE_UNIFORM, 1, x.size, 1, orc.F8_VIA_F16)
    h = x.astype(np.float16)                       # numpy: IEEE RNE
    assert np.array_equal(via, f16_to_f8_ref[h.view(np.uint16)])
    direct = orc.quantize(x, orc.F32, orc.F8E4M3FN, one, orc.SCALE_UNIFORM, 1, x.size)
    frac = np.count_nonzero(via != direct) / x.size
    assert 1e-4 < frac < 2e-2, frac                # the two policies do differ, on a small fraction
    # f16-representable inputs: one rounding either way
    hx = h.astype(np.float32)
    assert np.array_equal(orc.quantize(hx, orc.F32, orc.F8E4M3FN, one, orc.SCALE_UNIFORM, 1, hx.size, 1, orc.F8_VIA_F16),
                          orc.quantize(hx, orc.F32, orc.F8E4M3FN, one, orc.SCALE_UNIFORM, 1, hx.size))


def test_dequantize_closed_form(orc):
    g = rng(4)
    d0, d1 = 16, 24
    q = g.integers(-128, 128, (d0, d1)).astype(np.int8)
    sb = g.uniform(0.005, 0.02, (d0 // 4, d1)).astype(np.float32)
    y = orc.dequantize(q, orc.I8, orc.F32, sb.ravel(), orc.SCALE_COL, d0, d1, 4)
    assert np.array_equal(y.reshape(d0, d1), q.astype(np.float32) * np.repeat(sb, 4, axis=0))
    y16 = orc.dequantize(q, orc.I8, orc.F16, sb.ravel(), orc.SCALE_COL, d0, d1, 4)
    expect16 = (q.astype(np.float32) * np.repeat(sb, 4, axis=0)).astype(np.float16).view(np.uint16)
    assert np.array_equal(y16.reshape(d0, d1), expect16)
    codes = np.arange(256, dtype=np.uint8)
    y8 = orc.dequantize(codes, orc.F8E4M3FN, orc.F32, [np.float32(0.5)], orc.SCALE_UNIFORM, 1, 256)
    w = orc.widen(codes, orc.F8E4M3FN)
    ok = ~np.isnan(w)
    assert np.array_equal(y8[ok], w[ok] * np.float32(0.5))
    # reference block fixture raise-qdq-block-dequantize.mlir:5-13 uses an all-2 i4 tensor and equal
    # scale rows, for which contiguous and interleaved block layouts agree: [[1,1.2,1.4,1.6]] * 4 rows
    s = np.float32([[0.5, 0.6, 0.699999988, 0.8], [0.5, 0.6, 0.699999988, 0.8]])
    y = orc.dequantize(np.full(16, 2, dtype=np.uint8), orc.I4, orc.F32, s.ravel(), orc.SCALE_COL, 4, 4, 2)
    assert np.array_equal(y.reshape(4, 4), np.float32(2) * np.tile(s[0], (4, 1)))


def test_tripy_and_jax_value_tests(orc):
    """tripy/tests/integration/test_quantize.py:32-43,58-69 and
    mlir-tensorrt/integrations/PJRT/test/JAX/CustomPrimitives/test_quantize.py:60-83."""
    q = orc.quantize(np.float32([1.0, 2.0]), orc.F32, orc.I8, [np.float32(0.5)], orc.SCALE_UNIFORM, 1, 2)
    assert list(q) == [2, 4]
    q = orc.quantize(np.float32([[1, 2], [3, 4]]), orc.F32, orc.I8, np.float32([0.2, 0.1]), orc.SCALE_ROW, 2, 2, 2)
    assert list(q) == [5, 10, 30, 40]
    x = np.float32([[10, 20, 30, 40], [50, 60, 70, 80]])
    assert list(orc.quantize(x, orc.F32, orc.I8, [np.float32(1)], orc.SCALE_UNIFORM, 2, 4)) == [10, 20, 30, 40, 50, 60, 70, 80]
    assert list(orc.quantize(x, orc.F32, orc.I8, np.float32([2, 10]), orc.SCALE_ROW, 2, 4, 2)) == [5, 10, 15, 20, 5, 6, 7, 8]
    q = orc.quantize(x, orc.F32, orc.F8E4M3FN, np.float32([[1, 1, 1, 1]]).ravel(), orc.SCALE_COL, 2, 4, 2)
    assert list(orc.widen(q, orc.F8E4M3FN)) == [10, 20, 30, 40, 48, 60, 72, 80]   # f8 has 3 mantissa bits: 50->48, 70->72
    # int4 quantize->dequantize of ones with unit scales is the identity in every mode (test_qdq_int4)
    ones = np.ones((4, 4), dtype=np.float32)
    for kind, sc, nb in ((orc.SCALE_COL, np.ones(8, np.float32), 2), (orc.SCALE_UNIFORM, np.ones(1, np.float32), 1),
                         (orc.SCALE_ROW, np.ones(4, np.float32), 4), (orc.SCALE_COL, np.ones(4, np.float32), 4)):
        q = orc.quantize(ones, orc.F32, orc.I4_PACKED, sc, kind, 4, 4, nb)
        assert np.array_equal(orc.dequantize(q, orc.I4_PACKED, orc.F32, sc, kind, 4, 4, nb), ones.ravel())


def test_layernorm_and_softmax_against_torch_float64(orc):
    import torch
    g = rng(5)
    rows, d = 12, 384
    x = g.standard_normal((rows, d), dtype=np.float32)
    gamma = g.uniform(0.5, 1.5, d).astype(np.float32)
    beta = (g.standard_normal(d) * 0.1).astype(np.float32)
    y = orc.layernorm(x, gamma, beta, orc.F32, rows, d, 1e-5).reshape(rows, d)
    ref = torch.nn.functional.layer_norm(torch.from_numpy(x).double(), (d,), torch.from_numpy(gamma).double(),
                                         torch.from_numpy(beta).double(), 1e-5).numpy()
    assert np.max(np.abs(y - ref)) < 5e-6
    # eps sits inside the square root: with a constant row the output is exactly beta
    yc = orc.layernorm(np.full((1, d), 3.0, np.float32), gamma, beta, orc.F32, 1, d, 1e-5)
    assert np.array_equal(yc, beta)
    s = orc.softmax(x * 2, orc.F32, rows, d).reshape(rows, d)
    ref = torch.softmax(torch.from_numpy(x * 2).double(), dim=-1).numpy()
    assert np.max(np.abs(s - ref) / ref) < 5e-6
    assert np.allclose(s.sum(axis=1), 1.0, atol=1e-5)
    # narrow I/O goes through the pinned conversions
    xb = orc.narrow(x, orc.BF16)
    yb = orc.layernorm(xb, orc.narrow(gamma, orc.BF16), orc.narrow(beta, orc.BF16), orc.BF16, rows, d, 1e-5)
    refb = torch.nn.functional.layer_norm(torch.from_numpy(orc.widen(xb, orc.BF16)).double().reshape(rows, d), (d,),
                                          torch.from_numpy(orc.widen(orc.narrow(gamma, orc.BF16), orc.BF16)).double(),
                                          torch.from_numpy(orc.widen(orc.narrow(beta, orc.BF16), orc.BF16)).double(), 1e-5).numpy()
    assert np.max(np.abs(orc.widen(yb, orc.BF16).reshape(rows, d) - refb)) < 2.0 ** -7 * 4


def test_int8_gemm_is_exact_and_epilogue_order(orc):
    g = rng(6)
    M, K, N = 9, 70, 13                                       # non-square: a transposed operand cannot pass
    a = np.clip(np.rint(g.standard_normal((M, K)) * 40), -128, 127).astype(np.int8)
    w = np.clip(np.rint(g.standard_normal((K, N)) * 40), -128, 127).astype(np.int8)
    acc = orc.gemm_i8_i32(a, w)
    assert np.array_equal(acc, (a.astype(np.int64) @ w.astype(np.int64)).astype(np.int32))
    a_s = g.uniform(0.005, 0.02, M).astype(np.float32)
    w_s = g.uniform(0.005, 0.02, N).astype(np.float32)
    y = orc.gemm_w8a8(a, w, a_s, w_s)
    expect = ((acc.astype(np.float32) * a_s[:, None]) * w_s[None, :]).astype(np.float16).view(np.uint16)
    assert np.array_equal(y, expect)
    part = orc.gemm_w8a8(a, w, a_s, w_s, m0=3, mcount=4)
    assert np.array_equal(part, expect[3:7])
    # extreme accumulations stay inside int32: K * 128 * 128 for K = 4096 is 2^26
    big = orc.gemm_i8_i32(np.full((1, 4096), -128, np.int8), np.full((4096, 1), -128, np.int8))
    assert int(big[0, 0]) == 4096 * 128 * 128


def test_w4a16_dequant_and_accumulate(orc):
    g = rng(7)
    M, K, N, B = 5, 256, 24, 128
    a = orc.narrow(g.standard_normal((M, K), dtype=np.float32), orc.F16)
    w = g.integers(-8, 8, (K, N)).astype(np.int8)
    s = orc.narrow(g.uniform(0.005, 0.02, (K // B, N)).astype(np.float32), orc.F16)
    y = orc.gemm_w4a16(a, orc.pack_int4(w), s, K, N, B)
    wd = (w.astype(np.float16) * np.repeat(s.view(np.float16), B, axis=0))        # f16 multiply, one rounding
    ref = a.view(np.float16).astype(np.float64) @ wd.astype(np.float64)
    got = y.view(np.float16).astype(np.float64)
    assert np.max(np.abs(got - ref)) <= 1e-3 * np.max(np.abs(ref)) + 2.0 ** -11 * np.max(np.abs(ref))
    # one-hot activations read back single dequantized weights exactly: pins nibble order and block index
    eye = np.zeros((K, K), dtype=np.float32)
    np.fill_diagonal(eye, 1.0)
    yw = orc.gemm_w4a16(orc.narrow(eye, orc.F16), orc.pack_int4(w), s, K, N, B)
    assert np.array_equal(yw, wd.view(np.uint16))
