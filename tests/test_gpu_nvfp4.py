"""NVFP4 block quantize / dequantize on the GPU against the CPU oracle, through the C ABI.
Bar: codes, block scales and dequantized values BIT-EXACT (every step is a single correctly rounded
f32 op or an exact / RNE conversion)."""
import numpy as np
import pytest

from helpers import bits16, rng

pytestmark = pytest.mark.gpu


def _run(pkg, orc, x_f32, dname, amax=None, axis=-1):
    import torch
    o_dt = {"f32": orc.F32, "f16": orc.F16, "bf16": orc.BF16}[dname]
    t_dt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[dname]
    shape = x_f32.shape
    d1 = shape[-1]
    d0 = x_f32.size // d1
    store = orc.narrow(x_f32.ravel(), o_dt) if dname != "f32" else x_f32.ravel().copy()
    if dname == "f32":
        x = torch.from_numpy(store.reshape(shape)).cuda()
    else:
        x = torch.from_numpy(store.view(np.int16).reshape(shape)).view(t_dt).cuda()
    if amax is None:
        a_dev, _ = pkg.amax(x, 1.0)
        a_dev = a_dev.reshape(())
        amax = float(a_dev.item())
        assert np.float32(amax) == orc.amax(store, o_dt)
    else:
        a_dev = torch.tensor(amax, dtype=torch.float32, device="cuda")
    ba = 1 if axis == -1 else 0
    q, s = pkg.nvfp4_quantize(x, a_dev.clone(), axis=axis)
    q_ref, s_ref = orc.nvfp4_quantize(store, o_dt, amax, d0, d1, block_axis=ba)
    assert np.array_equal(s.cpu().numpy().ravel(), s_ref), "block scales (%s)" % pkg.last_kernel()
    assert np.array_equal(q.cpu().numpy(), q_ref), "codes (%s)" % pkg.last_kernel()
    y = pkg.nvfp4_dequantize(q, s, a_dev.clone(), t_dt, shape, axis=axis)
    y_ref = orc.nvfp4_dequantize(q_ref, s_ref, amax, o_dt, d0, d1, block_axis=ba)
    got = y.cpu().numpy().ravel().view(np.uint32) if dname == "f32" else bits16(y)
    ref = y_ref.view(got.dtype)
    # a NaN result (tensor amax 0: 0 * NaN) must be NaN on both sides; sign and payload of a NaN are not compared
    nan_ref = np.isnan(orc.widen(y_ref, o_dt)) if dname != "f32" else np.isnan(y_ref)
    nan_got = np.isnan(y.float().cpu().numpy().ravel())
    assert np.array_equal(nan_ref, nan_got)
    assert np.array_equal(got[~nan_ref], ref[~nan_ref]), "dequantized values (%s)" % pkg.last_kernel()
    return y


@pytest.mark.parametrize("dname", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", [(1, 16), (3, 64), (2, 128, 16), (1, 7, 100, 32), (5, 4112), (64, 2048), (2, 256, 32, 128)])
def test_reference_shapes(pkg, orc, dname, shape):
    """Shapes of mlir-tensorrt/integrations/PJRT/test/JAX/test_q_dq_nvfp4.py:96 and ragged wave spans."""
    x = rng(26 + len(shape)).standard_normal(shape).astype(np.float32)
    y = _run(pkg, orc, x, dname)
    xs = x if dname == "f32" else None
    if xs is not None:   # the reference test's acceptance bound
        assert np.all(np.abs(y.cpu().numpy() - x) <= 0.2 + 0.25 * np.abs(x))


@pytest.mark.parametrize("dname", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape", [(16, 8), (32, 64), (2, 48, 1000), (4096, 264), (3, 5, 160, 24)])
def test_blocks_along_the_second_to_last_axis(pkg, orc, dname, shape):
    """The op's other axis choice: blocks of 16 rows, scales [.., rows/16, cols]; with zero blocks, a block whose
    scale underflows, negative zeros and an outlier."""
    x = (rng(41 + len(shape)).standard_normal(shape) * 1.5).astype(np.float32)
    flat = x.reshape(-1, shape[-2], shape[-1])
    flat[0, :16, 0] = 0.0
    flat[0, :16, 1] *= 1e-7
    flat[0, 3, 1] = 0.0
    flat[-1, -16:, -1] = -0.0
    flat[0, 5, 2] = 700.0
    y = _run(pkg, orc, x, dname, axis=-2)
    assert y.shape == x.shape


def test_every_f16_value_through_the_f4_conversion(pkg, orc):
    """Blocks built so that S_enc_x is exactly 1 (tensor amax 6, one element of 6.0 per block): the other
    15 elements sweep every f16 value of magnitude <= 6, so the device's f16 -> f4 step is compared with
    the reference table on all of them, ties included."""
    h = np.arange(1 << 16, dtype=np.uint16)
    v = h.view(np.float16).astype(np.float32)
    v = v[np.isfinite(v) & (np.abs(v) <= 6.0)]
    pad = (-len(v)) % 15
    v = np.concatenate([v, np.zeros(pad, np.float32)]).reshape(-1, 15)
    x = np.concatenate([np.full((v.shape[0], 1), 6.0, np.float32), v], axis=1)
    _run(pkg, orc, x, "f32", amax=6.0)
    _run(pkg, orc, x, "f16", amax=6.0)


def test_zero_blocks_outliers_and_tiny_blocks(pkg, orc):
    g = rng(3)
    x = (g.standard_normal((64, 256)) * 2).astype(np.float32)
    x[3] = 0.0                                  # zero blocks: scale byte 0, codes 0
    x[5, 16:32] = 0.0
    x[7, :16] *= 1e-6                           # block whose scale underflows in e4m3: S_enc_x = inf -> +-6 and 0
    x[7, 3] = 0.0
    x[9, 40] = 900.0                            # outlier sets the tensor amax
    x[11, 100:116] = -0.0
    for d in ("f32", "bf16", "f16"):
        _run(pkg, orc, x, d)
    _run(pkg, orc, np.zeros((2, 64), np.float32), "f32")    # amax 0: every scale byte the e4m3 NaN, codes 0


def _f8_positive_values():
    """every finite non-negative f8E4M3FN value (OCP: bias 7, no infinities, 0x7F is NaN)"""
    out = []
    for b in range(0x7F):
        e, m = b >> 3, b & 7
        out.append(m * 2.0 ** -9 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7))
    return np.array(out, np.float32)


def test_block_maxima_whose_sixth_sits_on_a_scale_tie(pkg, orc):
    """Tensor amax 2688 makes S_enc exactly 1, so a block's scale byte is f8(RN(max / 6)): block maxima are placed so that
    max / 6 lands on, just below and just above every midpoint between neighbouring f8 values, where one ulp of the
    quotient changes the byte.  A second tensor walks maxima across 2^-125, where the kernel's short division hands
    over to the IEEE divide, with a tensor amax small enough that those quotients (f32 denormals) still give ordinary
    scale bytes."""
    f8 = _f8_positive_values()
    mid = (f8[:-1].astype(np.float64) + f8[1:].astype(np.float64)) / 2
    maxima = []
    for m in mid:
        q = np.float32(m)
        for k in range(-3, 4):
            t = q
            for _ in range(abs(k)):
                t = np.nextafter(t, np.float32(np.inf if k > 0 else 0), dtype=np.float32)
            x = np.float32(np.float64(t) * 6.0)
            for j in range(-2, 3):
                v = x
                for _ in range(abs(j)):
                    v = np.nextafter(v, np.float32(np.inf if j > 0 else 0), dtype=np.float32)
                maxima.append(v)
    maxima = np.array(maxima, np.float32)
    maxima = maxima[maxima <= 2688.0]
    maxima = maxima[:len(maxima) // 8 * 8]              # whole vectors of columns for the second-to-last-axis form
    x = np.zeros((len(maxima), 16), np.float32)
    x[:, 0] = maxima
    x[:, 5] = -maxima / 3
    for d in ("f32", "f16", "bf16"):       # the 16-bit forms round the maxima first: other quotients, same rule
        _run(pkg, orc, x, d, amax=2688.0)
    _run(pkg, orc, x.T.copy().reshape(16, -1), "f32", amax=2688.0, axis=-2)

    g = rng(77)
    bits = np.concatenate([np.arange(0x00FFFF00, 0x01000100, dtype=np.uint32),                 # across 2^-125
                           g.integers(0x00000001, 0x03000000, 6000, dtype=np.uint32)])          # denormals to 2^-121
    tiny = bits.view(np.float32)[:len(bits) // 8 * 8]
    x = np.zeros((len(tiny), 16), np.float32)
    x[:, 3] = tiny
    x[:, 9] = -tiny / 2
    _run(pkg, orc, x, "f32", amax=float(np.float32(2.0 ** -115)))
    _run(pkg, orc, x.T.copy().reshape(16, -1), "f32", amax=float(np.float32(2.0 ** -115)), axis=-2)


def test_nan_elements_and_an_overflowing_block_scale(pkg, orc):
    """NaN products take code 0 by the reference's rule wherever they come from: a NaN element of an ordinary block
    (the block maximum ignores it), and zeros of a block whose S_enc / f32(scale byte) overflows to infinity because
    the tensor amax is tiny."""
    g = rng(12)
    x = g.standard_normal((32, 64)).astype(np.float32)
    x[2, 5] = np.nan
    x[2, 40] = -np.nan
    x[7, 16:32] = np.nan                         # a whole block of NaN: maximum 0, scale byte 0
    x = np.clip(x, -4.0, 4.0)                    # the tensor amax handed over below bounds every block (NaN stays)
    for d in ("f32", "f16", "bf16"):
        _run(pkg, orc, x, d, amax=4.0)
        _run(pkg, orc, x, d, amax=4.0, axis=-2)
    z = np.zeros((8, 64), np.float32)
    z[:, ::7] = (g.standard_normal((8, 10)) * 2.0 ** -118).astype(np.float32)
    _run(pkg, orc, z, "f32", amax=float(np.float32(2.0 ** -116)))
    _run(pkg, orc, z.reshape(32, 16), "f32", amax=float(np.float32(2.0 ** -116)), axis=-2)


def test_c3_sized_tensor(pkg, orc):
    """bf16 [2048, 8192] (an eighth of BASELINE config 3's tensor, heavy-tail outliers): full bit-exact compare."""
    g = rng(3)
    x = (g.standard_normal((2048, 8192)) * np.sqrt(2.0)).astype(np.float32)
    x[g.random(x.shape) < 1e-3] *= 50.0
    orc.set_threads(16)
    try:
        _run(pkg, orc, x, "bf16")
    finally:
        orc.set_threads(1)


def test_argument_checks(pkg):
    import torch
    L = pkg.lib()
    t = torch.zeros(64, device="cuda")
    p = t.data_ptr()
    assert L.mtrt_hip_nvfp4_quantize(None, p, pkg.F32, p, p, p, 2, 24, 1) == 1
    assert b"divisible by 16" in L.mtrt_hip_last_error()
    assert L.mtrt_hip_nvfp4_quantize(None, p, pkg.F32, p, p, p, 24, 16, 0) == 1     # blocked extent 24
    assert L.mtrt_hip_nvfp4_quantize(None, p, pkg.F32, p, p, p, 16, 6, 0) == 1      # last extent not whole vectors
    assert L.mtrt_hip_nvfp4_quantize(None, p, pkg.F32, p, p, p, 16, 16, 2) == 1
    assert b"invalid axis" in L.mtrt_hip_last_error()
    assert L.mtrt_hip_nvfp4_quantize(None, p, pkg.I8, p, p, p, 2, 16, 1) == 1
    assert L.mtrt_hip_nvfp4_quantize(None, p + 4, pkg.F32, p, p, p, 2, 16, 1) == 1
    assert L.mtrt_hip_nvfp4_quantize(None, p, pkg.F32, p, p, None, 2, 16, 1) == 1
    assert L.mtrt_hip_nvfp4_dequantize(None, p, p, p, p, pkg.F32, 0, 16, 1) == 0
