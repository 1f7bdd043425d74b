"""Pins for the NVFP4 part of the CPU oracle (no GPU).

What fixes each piece:
  * f16 -> f4E2M1FN: an independent nearest-value search over the eight magnitudes with ties to the even
    code, on ALL 65536 f16 patterns, plus the cases the executor's expansion spells out
    (mlir-tensorrt/executor/lib/Passes/ExpandOps.cpp:555-640: 0.25 -> 0, 0.75 -> 1.0, 1.25 -> 1.0,
    1.75 -> 2.0, 2.5 -> 2.0, 3.5 -> 4.0, 5.0 -> 4.0, > 6 and inf -> +-6, NaN -> 0, +-0 -> code 0).
  * f4E2M1FN -> f32: the value table of the format (ExpandOps.cpp:365-461).
  * the block program: a float64/numpy restatement of
    mlir-tensorrt/integrations/PJRT/test/JAX/test_q_dq_nvfp4.py:21-45 with numpy float32 ops and the
    already pinned e4m3 conversion; the identity case (values on the f4 grid, amax 6); and that test's own
    acceptance bound (|dq(q(x)) - x| <= 0.2 + 0.25 |x|) on its shapes.
TensorRT's IDynamicQuantize itself is closed: parity against it is unpinned."""
import numpy as np
import pytest

from helpers import rng

MAGS = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])


def _nearest_even_code(v):
    if np.isnan(v):
        return 0
    a = abs(v)
    if a > 6:
        code = 7
    else:
        d = np.abs(MAGS - a)
        cands = np.flatnonzero(d == d.min())
        code = int(cands[0]) if len(cands) == 1 else int([c for c in cands if c % 2 == 0][0])
    return code | (8 if np.signbit(v) else 0)


def test_f16_to_f4_all_patterns(orc):
    L = orc.lib()
    for h in range(1 << 16):
        v = float(np.uint16(h).view(np.float16))
        assert L.orc_f16_to_f4e2m1fn(h, orc.IEEE) == _nearest_even_code(v), hex(h)


def test_f16_to_f4_reference_cases(orc):
    L = orc.lib()
    f16 = lambda x: int(np.float16(x).view(np.uint16))
    for x, code in [(0.25, 0), (0.2503, 1), (0.5, 1), (0.75, 2), (1.25, 2), (1.26, 3), (1.75, 4), (2.5, 4), (3.5, 6),
                    (5.0, 6), (5.01, 7), (6.0, 7), (1000.0, 7), (np.inf, 7), (-np.inf, 15), (-3.0, 13), (np.nan, 0)]:
        assert L.orc_f16_to_f4e2m1fn(f16(x), orc.REFHOST) == code, x
    # the expansion tests for zero before it applies the sign: +-0 -> code 0, a negative subnormal -> -0
    assert L.orc_f16_to_f4e2m1fn(0x8000, orc.REFHOST) == 0 and L.orc_f16_to_f4e2m1fn(0x8001, orc.REFHOST) == 8
    assert L.orc_f16_to_f4e2m1fn(0x8000, orc.IEEE) == 8
    for c in range(16):
        assert L.orc_f4e2m1fn_to_f32(c) == (-1.0 if c & 8 else 1.0) * MAGS[c & 7]


def _numpy_program(x, tensor_amax, orc):
    """test_q_dq_nvfp4.py:21-45 with numpy float32 scalars."""
    f = np.float32
    blocks = x.reshape(-1, 16).astype(np.float32)
    s_enc = f(2688.0) / f(tensor_amax)
    codes, scales, deq = [], [], []
    s_dec = f(tensor_amax) / f(2688.0)
    for b in blocks:
        s_dec_x = f(np.max(np.abs(b))) / f(6.0)
        s8 = orc.lib().orc_f32_to_f8e4m3fn(float(f(s_dec_x * s_enc)), orc.IEEE)
        s8f = f(orc.lib().orc_f8e4m3fn_to_f32(s8))
        with np.errstate(divide="ignore", invalid="ignore"):
            s_enc_x = f(s_enc / s8f)
            h = (b * s_enc_x).astype(np.float32).astype(np.float16)
        c = [_nearest_even_code(float(v)) for v in h]
        codes.append(c)
        scales.append(s8)
        deq.append([f(MAGS[k & 7] * (-1 if k & 8 else 1)) * f(s8f * s_dec) for k in c])
    return np.array(codes, np.uint8), np.array(scales, np.uint8), np.array(deq, np.float32)


@pytest.mark.parametrize("shape", [(1, 16), (3, 64), (2, 128, 16), (1, 7, 100, 32)])
def test_block_program_against_numpy(orc, shape):
    x = rng(26).standard_normal(shape).astype(np.float32)
    amax = np.float32(np.abs(x).max())
    d1 = shape[-1]
    d0 = x.size // d1
    q, s = orc.nvfp4_quantize(x, orc.F32, amax, d0, d1)
    codes, scales, deq = _numpy_program(x, amax, orc)
    packed = (codes[:, 0::2] | (codes[:, 1::2] << 4)).ravel()
    assert np.array_equal(q, packed) and np.array_equal(s, scales)
    y = orc.nvfp4_dequantize(q, s, amax, orc.F32, d0, d1)
    assert np.array_equal(y.view(np.uint32), deq.ravel().view(np.uint32))
    # the acceptance bound of the reference's own test
    assert np.all(np.abs(y - x.ravel()) <= 0.2 + 0.25 * np.abs(x.ravel()))


def test_identity_on_the_f4_grid_and_zero_blocks(orc):
    x = np.array([[0, 0.5, 1, 1.5, 2, 3, 4, 6, -0.5, -1, -1.5, -2, -3, -4, -6, 0], [0] * 16], dtype=np.float32)
    q, s = orc.nvfp4_quantize(x, orc.F32, 6.0, 2, 16)
    assert list(s) == [0x7E, 0]                        # 448 for the full-range block, 0 for the zero block
    assert list(q[:8]) == [0x10, 0x32, 0x54, 0x76, 0xA9, 0xCB, 0xED, 0x0F] and not q[8:].any()
    y = orc.nvfp4_dequantize(q, s, 6.0, orc.F32, 2, 16)
    assert np.array_equal(y, x.ravel())
    # an all-zero tensor: S_enc is infinite, every scale byte is the e4m3 NaN, every code 0
    q, s = orc.nvfp4_quantize(np.zeros((1, 32), np.float32), orc.F32, 0.0, 1, 32)
    assert not q.any() and list(s) == [0x7F, 0x7F]


def test_blocks_along_the_other_axis_are_the_transposed_problem(orc):
    """Blocks along d0 of x equal blocks along d1 of x^T: pins the block and scale indexing of block_axis = 0
    against the (numpy-pinned) block_axis = 1 path, codes compared after unpacking."""
    def unpack(q, n):
        out = np.empty(n, np.uint8)
        out[0::2] = q & 0xF
        out[1::2] = q >> 4
        return out
    for d0, d1 in ((16, 3), (48, 10), (32, 64)):
        x = (rng(d0 + d1).standard_normal((d0, d1)) * 2).astype(np.float32)
        x[:16, 0] = 0.0
        amax = np.float32(np.abs(x).max())
        q0, s0 = orc.nvfp4_quantize(x, orc.F32, amax, d0, d1, block_axis=0)
        qt, st = orc.nvfp4_quantize(np.ascontiguousarray(x.T), orc.F32, amax, d1, d0, block_axis=1)
        assert np.array_equal(unpack(q0, d0 * d1).reshape(d0, d1), unpack(qt, d0 * d1).reshape(d1, d0).T)
        assert np.array_equal(s0.reshape(d0 // 16, d1), st.reshape(d1, d0 // 16).T)
        y0 = orc.nvfp4_dequantize(q0, s0, amax, orc.F32, d0, d1, block_axis=0)
        yt = orc.nvfp4_dequantize(qt, st, amax, orc.F32, d1, d0, block_axis=1)
        assert np.array_equal(y0.reshape(d0, d1), yt.reshape(d1, d0).T)
