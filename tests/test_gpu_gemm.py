"""Parity of the GEMM clusters with the CPU oracle, through the C ABI.

W8A8: the int32 accumulators are exact under any summation order and the epilogue is a
fixed chain of correctly rounded f32 operations followed by one f16 narrowing, so the
f16 outputs must be BIT-IDENTICAL to the oracle's.

W4A16: the dequantised weights are bit-exact (one f16 rounding, checked by reading them
back through one-hot activations, once per tile kernel); the f32 accumulation runs in the
matrix cores' order, not the host's left-to-right order, so outputs are compared under two bounds:
    against the oracle, every element:   |got - ref| <= 1 ulp_f16(ref) + noise
    against float64, every element:      |got - exact| <= 1e-3 * |exact| + 1 ulp_f16(exact) + noise
    noise = 1e-5 * sqrt(K) * rms(a_row) * rms(wd_col)
and the share of outputs whose bits differ from the oracle's is bounded (kMaxShare).  The noise term is the size of
the rounding error of a length-K f32 dot product (measured on the host at K = 4096: 0.7e-5 in these units); it is
what lets an output whose terms cancel to nearly zero be compared at all, and it is far below one f16 ulp of a
typical output, so a kernel that rounded once too often per product would not pass.
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
    # up to 64 rows take the kernels that read the weights once at these sizes
    assert kernel == ("mtrt_gemm_w8a8_nk_rows32" if M <= 32 else "mtrt_gemm_w8a8_nk_rows64" if M <= 64 else
                      "mtrt_gemm_w8a8_nk_rows128" if M <= 128 else "mtrt_gemm_w8a8_nk")
    assert np.array_equal(bits16(y).reshape(M, N), orc.gemm_w8a8(a, w, a_s, w_s))


@pytest.mark.parametrize("shape", [(1, 128, 32), (16, 4096, 11008), (32, 4096, 11008), (17, 384, 200), (9, 1280, 4099), (13, 640, 8240),
                                   (32, 256, 16384), (25, 512, 16400), (8, 2048, 8209), (16, 128, 40), (16, 4096, 4096), (32, 4096, 6144), (5, 8192, 8192), (3, 512, 65000), (2, 128, 200000)])
def test_w8a8_small_m_kernel_on_row_major_weights(pkg, orc, shape):
    """M <= 32 with [N,K] weights as they are: one workgroup per 32 weight rows, eight waves splitting K and reading
    whole rows; K = 128 and 384 leave waves without a slice, 640 and 1280 give them uneven shares; ragged last tiles
    whose missing rows repeat row N - 1; very wide weights stay on the tile loop.  Integer sums: bit-exact."""
    M, K, N = shape
    a, w, a_s, w_s = _w8a8_inputs(rng(M + K + N), M, K, N)
    print("case: w8a8 small M, row-major weights", shape, flush=True)
    y, kernel = _run_w8a8(pkg, a, w, a_s, w_s)
    # the kernel that reads the weights once, or the tile loop where the host's estimate puts very wide weights
    assert kernel in ("mtrt_gemm_w8a8_nk_rows32", "mtrt_gemm_w8a8_nk")
    orc.set_threads(16)
    ref = orc.gemm_w8a8(a, w, a_s, w_s)
    orc.set_threads(1)
    assert np.array_equal(bits16(y).reshape(M, N), ref)


@pytest.mark.parametrize("shape", [(64, 512, 4096), (33, 1024, 520), (50, 256, 8209), (64, 4096, 4100), (41, 128, 31),
                                   (128, 512, 4096), (65, 1024, 520), (100, 256, 8209), (128, 4096, 1030), (97, 128, 31)])
def test_w8a8_33_to_128_rows_on_row_major_weights(pkg, orc, shape):
    """Two (up to 64 rows) or four (up to 128) activation row tiles against each weight fragment: every row of every
    tile, ragged M and N, waves with and without slices.  Integer sums: bit-exact."""
    M, K, N = shape
    a, w, a_s, w_s = _w8a8_inputs(rng(M + K + N), M, K, N)
    y, kernel = _run_w8a8(pkg, a, w, a_s, w_s)
    assert kernel == ("mtrt_gemm_w8a8_nk_rows64" if M <= 64 else "mtrt_gemm_w8a8_nk_rows128")
    assert np.array_equal(bits16(y).reshape(M, N), orc.gemm_w8a8(a, w, a_s, w_s))


# Up to 32 rows on fragment-order weights: the four-wave kernel with hand-counted waits (up to 16 rows) or the
# wave-private eight-wave kernel; which of the two depends on the number of compute units, the results do not.
_FRAG_SMALL = {"mtrt_gemm_w8a8_frag_rows32", "mtrt_gemm_w8a8_small16"}


def _frag_small_ok(kernel, M):
    return kernel in _FRAG_SMALL and (M <= 16 or kernel == "mtrt_gemm_w8a8_frag_rows32")


# the tile kernels on fragment-order weights (one launch in rounds of tiles, or one workgroup per compute unit walking
# its share of the columns)
_FRAG_TILE = {"mtrt_gemm_w8a8_frag", "mtrt_gemm_w8a8_frag_t256x384"}


def _run_w8a8_frag(pkg, a, w, a_s, w_s, from_nk=False):
    import torch
    ad, wd = torch.from_numpy(a).cuda(), torch.from_numpy(w).cuda()
    wf = pkg.gemm_w8a8_prepack_fragments(wd.t().contiguous(), is_nk=True) if from_nk else pkg.gemm_w8a8_prepack_fragments(wd)
    y = pkg.gemm_w8a8_fragments(ad, wf, torch.from_numpy(a_s).cuda(), torch.from_numpy(w_s).cuda(), w.shape[1])
    return y, pkg.last_kernel()


@pytest.mark.parametrize("shape", [(256, 128, 128), (512, 512, 256), (300, 256, 200), (1, 128, 1), (37, 384, 129),
                                   (257, 1024, 130), (700, 256, 8200), (2000, 128, 16416)])
def test_w8a8_weights_in_registers_kernel(pkg, orc, shape):
    """Full tiles, half-width tiles of a partial last round, ragged M and N, one slice and many."""
    M, K, N = shape
    a, w, a_s, w_s = _w8a8_inputs(rng(M + K + N), M, K, N)
    print("case: w8a8 fragments", shape, flush=True)
    y, kernel = _run_w8a8_frag(pkg, a, w, a_s, w_s, from_nk=(M % 2 == 1))
    assert (_frag_small_ok(kernel, M) if M <= 32 else kernel in ("mtrt_gemm_w8a8_frag_rows64", "mtrt_gemm_w8a8_frag") if M <= 64
            else kernel in _FRAG_TILE), kernel
    orc.set_threads(16)
    ref = orc.gemm_w8a8(a, w, a_s, w_s)
    orc.set_threads(1)
    assert np.array_equal(bits16(y).reshape(M, N), ref)


@pytest.mark.parametrize("shape", [(1, 128, 32), (16, 4096, 11008), (32, 4096, 11008), (17, 384, 200), (9, 1280, 4099), (13, 640, 8240),
                                   (32, 256, 16384), (25, 512, 16400), (8, 2048, 8209), (16, 128, 40)])
def test_w8a8_small_m_kernel(pkg, orc, shape):
    """M <= 32: one workgroup per 32-column tile with four or eight waves splitting K.  K = 128 and 384 leave waves without a
    slice, 1280 gives them 2 or 3 (only the one-at-a-time tail), 4096 eight (two groups of four); N = 11008 gives 344
    tiles (one workgroup per compute unit, the first 88 with two tiles), 16384 two each, 16400 and 8209 one tile beyond
    those forms; ragged last tiles; M = 8 stays at one tile per workgroup.  Integer sums: bit-exact."""
    M, K, N = shape
    a, w, a_s, w_s = _w8a8_inputs(rng(M + K + N), M, K, N)
    y, kernel = _run_w8a8_frag(pkg, a, w, a_s, w_s, from_nk=(M % 2 == 1))
    assert _frag_small_ok(kernel, M), kernel
    orc.set_threads(16)
    ref = orc.gemm_w8a8(a, w, a_s, w_s)
    orc.set_threads(1)
    assert np.array_equal(bits16(y).reshape(M, N), ref)


@pytest.mark.parametrize("shape", [(64, 512, 4100), (50, 256, 8192), (33, 1024, 520), (64, 4096, 4096), (41, 128, 31), (48, 4096, 11008),
                                   (128, 512, 4096), (65, 1024, 520), (100, 256, 8209), (128, 4096, 1030), (97, 128, 31), (96, 4096, 11008),
                                   (40, 128, 150000)])
def test_w8a8_33_to_128_rows_on_fragment_order_weights(pkg, orc, shape):
    """Two (up to 64 rows) or four activation row tiles against weight fragments that go from memory straight into
    registers: every row of every tile, ragged M and N (the re-layout holds zeros past N), waves with and without
    slices; shapes whose estimate favours the tile launch stay there.  Integer sums: bit-exact."""
    M, K, N = shape
    a, w, a_s, w_s = _w8a8_inputs(rng(M + K + N), M, K, N)
    print("case: w8a8 fragments, 33..128 rows", shape, flush=True)
    y, kernel = _run_w8a8_frag(pkg, a, w, a_s, w_s, from_nk=(M % 2 == 1))
    assert kernel in (("mtrt_gemm_w8a8_frag_rows64" if M <= 64 else "mtrt_gemm_w8a8_frag_rows128"),) + tuple(_FRAG_TILE), kernel
    orc.set_threads(16)
    ref = orc.gemm_w8a8(a, w, a_s, w_s)
    orc.set_threads(1)
    assert np.array_equal(bits16(y).reshape(M, N), ref)


@pytest.mark.parametrize("shape", [(5, 7, 3), (33, 100, 65), (2, 130, 4), (300, 1, 140), (129, 15, 257), (128, 16, 128), (130, 271, 131),
                                   (64, 4100, 520), (257, 1153, 385), (100, 4160, 264)])
def test_w8a8_any_k_kernel(pkg, orc, shape):
    """K that is not a whole number of 128-byte slices: the 128 x 128 tile kernel with byte-aligned loads and a
    zero-padded last k-step.  K below one chunk, one byte over a chunk / a k-step, several k-steps, ragged M and N,
    several tiles per axis.  Integer sums: bit-exact."""
    M, K, N = shape
    a, w, a_s, w_s = _w8a8_inputs(rng(M * K + N), M, K, N)
    print("case: w8a8 any K", shape, flush=True)
    y, kernel = _run_w8a8(pkg, a, w, a_s, w_s)
    assert kernel == "mtrt_gemm_w8a8_nk_edge"
    assert np.array_equal(bits16(y).reshape(M, N), orc.gemm_w8a8(a, w, a_s, w_s))


def test_w8a8_operands_off_alignment_and_outputs_inside_a_larger_buffer(pkg, orc):
    """Operands one and three bytes off 16-byte alignment with K a multiple of 128, an output one element off 4-byte
    alignment: same kernel, nothing written outside y."""
    import torch
    M, K, N = 200, 256, 136
    a, w, a_s, w_s = _w8a8_inputs(rng(77), M, K, N)
    abuf = torch.zeros(M * K + 16, dtype=torch.int8, device="cuda")
    wbuf = torch.zeros(N * K + 16, dtype=torch.int8, device="cuda")
    ybuf = torch.full((M * N + 9,), 7.0, dtype=torch.float16, device="cuda")
    ad, wd, yd = abuf[1:1 + M * K].view(M, K), wbuf[3:3 + N * K].view(N, K), ybuf[1:1 + M * N].view(M, N)
    ad.copy_(torch.from_numpy(a))
    wd.copy_(torch.from_numpy(np.ascontiguousarray(w.T)))
    pkg.gemm_w8a8(ad, wd, torch.from_numpy(a_s).cuda(), torch.from_numpy(w_s).cuda(), out=yd)
    assert pkg.last_kernel() == "mtrt_gemm_w8a8_nk_edge"
    assert np.array_equal(bits16(yd.contiguous()).reshape(M, N), orc.gemm_w8a8(a, w, a_s, w_s))
    assert float(ybuf[0]) == 7.0 and bool((ybuf[1 + M * N:] == 7.0).all())


def test_w8a8_empty_reduction_is_zero(pkg, orc):
    """K = 0: every sum is empty, the outputs are the scaled zero; the one-element-per-lane kernel."""
    M, K, N = 5, 0, 9
    a, w, a_s, w_s = _w8a8_inputs(rng(5), M, K, N)
    import torch
    y = pkg.gemm_w8a8(torch.from_numpy(a).cuda(), torch.zeros((N, 0), dtype=torch.int8, device="cuda"),
                      torch.from_numpy(a_s).cuda(), torch.from_numpy(w_s).cuda())
    assert pkg.last_kernel() == "mtrt_gemm_w8a8_nk_any"
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


def test_w8a8_tile_epilogue_over_the_whole_f16_range(pkg, orc):
    """Row scales from 2^-34 to 2^6 put the outputs of the tile kernels' epilogue (two f32 roundings, then a pair of f16
    conversions in one instruction) everywhere between f16 subnormals, ties at the subnormal boundary and overflow to
    infinity; the bits are the oracle's."""
    M, K, N = 320, 128, 416
    a, w, _, w_s = _w8a8_inputs(rng(61), M, K, N)
    a_s = (2.0 ** np.linspace(-34, 6, M)).astype(np.float32)
    for run in (_run_w8a8, _run_w8a8_frag):
        y, kernel = run(pkg, a, w, a_s, w_s)
        got = bits16(y).reshape(M, N)
        ref = orc.gemm_w8a8(a, w, a_s, w_s)
        assert np.array_equal(got, ref), kernel
    f = ref.view(np.float16)
    assert np.isinf(f).any() and ((np.abs(f) < 6.0e-5) & (f != 0)).any()
    y = _launch_wide_w8a8(pkg, a, w, a_s, w_s)
    assert np.array_equal(bits16(y).reshape(M, N), ref)


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
    # the weights-in-registers kernel gives the same bits
    y2, kernel2 = _run_w8a8_frag(pkg, a, w, a_s, w_s)
    assert kernel2 in _FRAG_TILE
    assert torch.equal(y2, expect)


def _launch_wide_w8a8(pkg, a, w, a_s, w_s):
    """mtrt_gemm_w8a8_frag_t256x384 launched by hand from the built-in module (the entry point takes it only where its
    rounds come out shorter), with the grid its comment gives."""
    import ctypes
    import torch
    L = pkg.lib()
    pkg.check(L.mtrt_hip_init())
    M, K = a.shape
    N = w.shape[1]
    ad, wd = torch.from_numpy(a).cuda(), torch.from_numpy(w).cuda()
    wf = pkg.gemm_w8a8_prepack_fragments(wd)
    asd, wsd = torch.from_numpy(a_s).cuda(), torch.from_numpy(w_s).cuda()
    y = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    name = b"mtrt_gemm_w8a8_frag_t256x384"
    fn = L.mtrt_cuda_module_get_function(L.mtrt_hip_builtin_module(), name, len(name))
    assert fn
    vals = [ctypes.c_void_p(ad.data_ptr()), ctypes.c_void_p(wf.data_ptr()), ctypes.c_void_p(asd.data_ptr()), ctypes.c_void_p(wsd.data_ptr()),
            ctypes.c_void_p(y.data_ptr()), ctypes.c_int64(M), ctypes.c_int64(K), ctypes.c_int64(N)]
    args = (ctypes.c_void_p * len(vals))(*[ctypes.cast(ctypes.pointer(v), ctypes.c_void_p) for v in vals])
    tiles = ((M + 255) // 256) * ((N + 383) // 384)
    L.mtrt_cuda_launch_kernel(fn, 8 * ((tiles + 7) // 8), 1, 1, 256, 1, 1, 0, torch.cuda.current_stream().cuda_stream, args)
    torch.cuda.synchronize()
    return y


@pytest.mark.parametrize("shape", [(256, 128, 384), (1, 128, 1), (300, 256, 200), (257, 384, 385), (512, 1024, 1160), (700, 256, 8200),
                                   (130, 512, 4001), (2048, 128, 11008)])
def test_w8a8_wide_tile_kernel(pkg, orc, shape):
    """The 256 x 384 tile kernel on its own: one slice (K = 128: nothing but the first loads and the surplus ones), three
    slices, many; one tile and several rounds' worth; M and N that leave the last row and column tiles ragged, N that is
    not a whole vector (the element-wise stores), panels whose last waves have no column at all.  Integer sums: bit-exact."""
    M, K, N = shape
    a, w, a_s, w_s = _w8a8_inputs(rng(M + K + N + 1), M, K, N)
    print("case: w8a8 wide tile", shape, flush=True)
    y = _launch_wide_w8a8(pkg, a, w, a_s, w_s)
    orc.set_threads(16)
    ref = orc.gemm_w8a8(a, w, a_s, w_s)
    orc.set_threads(1)
    assert np.array_equal(bits16(y).reshape(M, N), ref)


def test_w8a8_wide_tile_kernel_equals_the_entry_point_on_random_shapes(pkg):
    """Integer sums are exact in any order, so whichever kernel the entry point picks for a shape (wave-private rows
    kernels, 256 x 256 tiles, half tiles) must give the wide tile kernel's bits: 24 seeded shapes with ragged M, N and
    one to sixteen slices."""
    import torch
    g = rng(2024)
    for case in range(24):
        M = int(g.integers(1, 1400))
        K = 128 * int(g.integers(1, 17))
        N = int(g.integers(1, 2600))
        a, w, a_s, w_s = _w8a8_inputs(g, M, K, N)
        print("case: w8a8 wide vs entry point", (M, K, N), flush=True)
        y_wide = _launch_wide_w8a8(pkg, a, w, a_s, w_s)
        y_api, kernel = _run_w8a8_frag(pkg, a, w, a_s, w_s)
        assert torch.equal(y_wide, y_api), ((M, K, N), kernel)


def test_w8a8_wide_tile_is_taken_where_its_rounds_are_shorter(pkg, orc):
    """At the shape of BASELINE config 4 (344 tiles of 256 x 256 = one and a half rounds on 256 compute units, 232 of
    256 x 384 = one) the entry point launches the wide kernel; the result is the oracle's either way."""
    import torch
    M, K, N = 2048, 256, 11008
    a, w, a_s, w_s = _w8a8_inputs(rng(44), M, K, N)
    y, kernel = _run_w8a8_frag(pkg, a, w, a_s, w_s)
    if torch.cuda.get_device_properties(0).multi_processor_count == 256:
        assert kernel == "mtrt_gemm_w8a8_frag_t256x384", kernel
    assert kernel in _FRAG_TILE
    orc.set_threads(16)
    ref = orc.gemm_w8a8(a, w, a_s, w_s)
    orc.set_threads(1)
    assert np.array_equal(bits16(y).reshape(M, N), ref)


def test_w8a8_argument_checks(pkg):
    import torch
    L = pkg.lib()
    t = torch.zeros(256, device="cuda")
    assert L.mtrt_hip_gemm_w8a8(None, t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), -1, 128, 4) == 1
    assert L.mtrt_hip_gemm_w8a8(None, None, t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), 4, 128, 4) == 1
    assert L.mtrt_hip_gemm_w8a8(None, t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), 0, 128, 4) == 0


# ---------------------------------------------------------------------------------------
# W4A16
# ---------------------------------------------------------------------------------------

def _w4a16_inputs(orc, g, M, K, N, B):
    a = orc.narrow(g.standard_normal((M, K), dtype=np.float32), orc.F16)
    w = g.integers(-8, 8, (K, N)).astype(np.int8)
    s = orc.narrow(g.uniform(0.005, 0.02, (K // B, N)).astype(np.float32), orc.F16)
    return a, w, orc.pack_int4(w), s


def _run_w4a16(pkg, a, wp_host, s, K, N, B, prepack=True):
    import torch
    ad = torch.from_numpy(a.view(np.int16)).view(torch.float16).cuda()
    wd = torch.from_numpy(wp_host).cuda()
    sd = torch.from_numpy(s.view(np.int16)).view(torch.float16).cuda()
    pre = pkg.gemm_w4a16_prepack(wd, K, N) if prepack else None
    y = pkg.gemm_w4a16(ad, sd, K, N, B, w_kn_packed=wd, w_prepacked=pre)
    return y, pkg.last_kernel()


kNoise = 1e-5        # f32 accumulation noise, in units of sqrt(K) * rms(a_row) * rms(wd_col)
kMaxShare = 0.015    # largest share of outputs that may differ from the oracle's bits, by one f16 ulp (measured: at
                     # most 0.61 %, 0.50 % at K = 4096: sums that land within the two orders' f32 difference of an f16 tie)


def _ulp16(v):
    return 2.0 ** np.floor(np.log2(np.maximum(np.abs(v), 2.0 ** -14))) * 2.0 ** -10


def _check_w4a16(orc, y, a, w, s, K, N, B, ref_bits, max_share=kMaxShare):
    got = bits16(y).reshape(-1, N).view(np.float16).astype(np.float64)
    ref = ref_bits.view(np.float16).astype(np.float64)
    af = a.view(np.float16).astype(np.float64)
    wdf = (w.astype(np.float16) * np.repeat(s.view(np.float16), B, axis=0)).astype(np.float64)
    exact = af @ wdf
    noise = kNoise * np.sqrt(K) * np.sqrt((af ** 2).mean(axis=1))[:, None] * np.sqrt((wdf ** 2).mean(axis=0))[None, :]
    for name, target, rel in (("oracle", ref, 0.0), ("float64", exact, 1e-3)):
        bound = rel * np.abs(target) + _ulp16(target) + noise
        err = np.abs(got - target)
        assert np.all(err <= bound), "%s: worst excess %g at %s" % (name, (err - bound).max(), np.unravel_index(np.argmax(err - bound), err.shape))
    share = np.count_nonzero(got != ref) / got.size
    print("w4a16: %d outputs, %.4f %% differ from the oracle's bits" % (got.size, 100.0 * share), flush=True)
    assert share <= max(max_share, 2.0 / got.size), "share of outputs that differ from the oracle: %g" % share
    return share


@pytest.mark.parametrize("shape", [(16, 256, 64), (1, 128, 32), (32, 1024, 96), (7, 512, 40), (33, 256, 64), (128, 512, 64),
                                   (200, 384, 100), (300, 1024, 256), (512, 256, 384), (48, 512, 1000), (64, 256, 96), (50, 384, 8209)])
def test_w4a16_small_shapes(pkg, orc, shape):
    M, K, N = shape
    B = 128
    a, w, wp, s = _w4a16_inputs(orc, rng(M + K + N), M, K, N, B)
    y, kernel = _run_w4a16(pkg, a, wp, s, K, N, B)
    # 33..64 rows run as two launches of the small-M kernels; the last one is that of the rows beyond 32
    last = M - 32 if 32 < M <= 64 else M
    assert kernel == ("mtrt_gemm_w4a16_strips16" if last <= 16 else "mtrt_gemm_w4a16_skinny" if last <= 32 else
                      "mtrt_gemm_w4a16_t128x64" if N <= 64 else "mtrt_gemm_w4a16_t128x128")
    _check_w4a16(orc, y, a, w, s, K, N, B, orc.gemm_w4a16(a, wp, s, K, N, B))


def test_w4a16_dequantised_weights_are_bit_exact(pkg, orc):
    """One-hot activations read the dequantised weights back unchanged: pins the prepack order,
    the nibble decoding, the block index of the scale and the single f16 rounding."""
    K, N, B = 512, 160, 128
    g = rng(31)
    w = g.integers(-8, 8, (K, N)).astype(np.int8)
    s = orc.narrow(g.uniform(0.005, 0.02, (K // B, N)).astype(np.float32), orc.F16)
    eye = np.zeros((K, K), np.float32)
    np.fill_diagonal(eye, 1.0)
    wd = (w.astype(np.float16) * np.repeat(s.view(np.float16), B, axis=0)).view(np.uint16)
    for rows in (slice(0, K), slice(0, 32), slice(100, 116)):        # big-tile, skinny (32 rows), skinny (16 rows)
        a = orc.narrow(eye[rows], orc.F16)
        y, kernel = _run_w4a16(pkg, a, orc.pack_int4(w), s, K, N, B)
        assert np.array_equal(bits16(y).reshape(-1, N), wd[rows]), kernel


@pytest.mark.parametrize("case", [(2048, 8192, "mtrt_gemm_w4a16_t256x256"), (512, 1024, "mtrt_gemm_w4a16_t128x128"),
                                  (2048, 11008, "mtrt_gemm_w4a16_t256x384"), (1536, 4096, "mtrt_gemm_w4a16_t128x256")])
def test_w4a16_tile_kernels_dequantise_bit_exactly(pkg, orc, case):
    """Identity activations (M = K) through the 256 x 384, 256 x 256, 128 x 256 and 128 x 128 tile kernels: every output is one product
    1 x wd plus zeros, so y must equal the dequantised weights bit for bit whatever the order of the sums: pins the
    fragment order of the re-laid weights, the nibble decoding, the scale row of every K block and the single f16
    rounding in the kernels that carry the benchmark."""
    K, N, want = case
    B = 128
    g = rng(K + N)
    w = g.integers(-8, 8, (K, N)).astype(np.int8)
    s = orc.narrow(g.uniform(0.005, 0.02, (K // B, N)).astype(np.float32), orc.F16)
    eye = np.zeros((K, K), np.float32)
    np.fill_diagonal(eye, 1.0)
    wd = (w.astype(np.float16) * np.repeat(s.view(np.float16), B, axis=0)).view(np.uint16)
    y, kernel = _run_w4a16(pkg, orc.narrow(eye, orc.F16), orc.pack_int4(w), s, K, N, B)
    import torch
    if torch.cuda.get_device_properties(0).multi_processor_count == 256:    # (the tile is chosen by rounds of the compute units)
        assert kernel == want
    assert np.array_equal(bits16(y).reshape(K, N), wd)


def _launch_wide_w4a16(pkg, a, wp_host, s, K, N, B):
    """mtrt_gemm_w4a16_t256x384 launched by hand from the built-in module (the entry point takes it only where its
    rounds come out shorter), with the grid its comment gives."""
    import ctypes
    import torch
    L = pkg.lib()
    pkg.check(L.mtrt_hip_init())
    M = a.shape[0]
    ad = torch.from_numpy(a.view(np.int16)).view(torch.float16).cuda()
    sd = torch.from_numpy(s.view(np.int16)).view(torch.float16).cuda()
    pre = pkg.gemm_w4a16_prepack(torch.from_numpy(wp_host).cuda(), K, N)
    y = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    name = b"mtrt_gemm_w4a16_t256x384"
    fn = L.mtrt_cuda_module_get_function(L.mtrt_hip_builtin_module(), name, len(name))
    assert fn
    vals = [ctypes.c_void_p(ad.data_ptr()), ctypes.c_void_p(pre.data_ptr()), ctypes.c_void_p(sd.data_ptr()), ctypes.c_void_p(y.data_ptr()),
            ctypes.c_int64(M), ctypes.c_int64(K), ctypes.c_int64(N), ctypes.c_int64(B)]
    args = (ctypes.c_void_p * len(vals))(*[ctypes.cast(ctypes.pointer(v), ctypes.c_void_p) for v in vals])
    tiles = ((M + 255) // 256) * ((N + 383) // 384)
    L.mtrt_cuda_launch_kernel(fn, 8 * ((tiles + 7) // 8), 1, 1, 256, 1, 1, 0, torch.cuda.current_stream().cuda_stream, args)
    torch.cuda.synchronize()
    return y


@pytest.mark.parametrize("case", [(256, 64, 384, 64), (1, 128, 1, 128), (300, 256, 200, 64), (257, 192, 385, 64), (512, 1024, 1160, 128),
                                  (700, 256, 8200, 256), (130, 512, 4001, 128)])
def test_w4a16_wide_tile_kernel(pkg, orc, case):
    """The 256 x 384 tile kernel on its own: one slice (K = 64), three, many; blocks of one slice and of several; one tile
    and several rounds' worth; ragged last row and column tiles, N that is not a whole vector, panels whose last waves
    have no column at all.  Against the oracle and float64 within the bound of the tile kernels."""
    M, K, N, B = case
    a, w, wp, s = _w4a16_inputs(orc, rng(M * K + N + 1), M, K, N, B)
    print("case: w4a16 wide tile", case, flush=True)
    y = _launch_wide_w4a16(pkg, a, wp, s, K, N, B)
    orc.set_threads(16)
    ref = orc.gemm_w4a16(a, wp, s, K, N, B)
    orc.set_threads(1)
    _check_w4a16(orc, y, a, w, s, K, N, B, ref)


def test_w4a16_wide_tile_kernel_equals_the_256_x_256_tile_on_random_shapes(pkg, orc):
    """Both 256-row tile kernels add a row's products in the same order (k ascending, one f32 accumulator per output),
    so their results are the same bits: 16 seeded shapes with ragged M and N, blocks of one to four slices.  (The
    entry point is steered to the 256 x 256 tile by launching it by hand, like the wide one.)"""
    import ctypes
    import torch
    L = pkg.lib()
    g = rng(2025)
    name = b"mtrt_gemm_w4a16_t256x256"
    fn = L.mtrt_cuda_module_get_function(L.mtrt_hip_builtin_module(), name, len(name))
    assert fn
    for case in range(16):
        M = int(g.integers(1, 1200))
        B = 64 * int(g.integers(1, 5))
        K = B * int(g.integers(1, 9))
        N = int(g.integers(1, 2400))
        a, w, wp, s = _w4a16_inputs(orc, g, M, K, N, B)
        print("case: w4a16 wide vs 256 x 256", (M, K, N, B), flush=True)
        y_wide = _launch_wide_w4a16(pkg, a, wp, s, K, N, B)
        ad = torch.from_numpy(a.view(np.int16)).view(torch.float16).cuda()
        sd = torch.from_numpy(s.view(np.int16)).view(torch.float16).cuda()
        pre = pkg.gemm_w4a16_prepack(torch.from_numpy(wp).cuda(), K, N)
        y = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
        vals = [ctypes.c_void_p(ad.data_ptr()), ctypes.c_void_p(pre.data_ptr()), ctypes.c_void_p(sd.data_ptr()), ctypes.c_void_p(y.data_ptr()),
                ctypes.c_int64(M), ctypes.c_int64(K), ctypes.c_int64(N), ctypes.c_int64(B)]
        args = (ctypes.c_void_p * len(vals))(*[ctypes.cast(ctypes.pointer(v), ctypes.c_void_p) for v in vals])
        tiles = ((M + 255) // 256) * ((N + 255) // 256)
        L.mtrt_cuda_launch_kernel(fn, 8 * ((tiles + 7) // 8), 1, 1, 256, 1, 1, 0, torch.cuda.current_stream().cuda_stream, args)
        torch.cuda.synchronize()
        assert torch.equal(y_wide.view(torch.int16), y.view(torch.int16)), (M, K, N, B)


@pytest.mark.parametrize("case", [(5, 48, 7, 16), (9, 100, 33, 20), (3, 128, 6, 128), (130, 256, 200, 32), (70, 192, 131, 16),
                                  (256, 520, 129, 8), (33, 77, 300, 7), (140, 1024, 257, 1024), (64, 4096, 130, 32), (3, 65, 1, 65), (4, 70, 3, 5), (2, 129, 7, 43)])
def test_w4a16_any_shape_kernel(pkg, orc, case):
    """Blocks that are not multiples of 64, K that is not, odd N (rows of nibbles that start in the middle of a byte),
    no re-laid weights: the 128 x 128 tile kernel that dequantises the original nibbles.  f32 sums in the matrix
    cores' order: within the bound of the tile kernels, against the oracle and against float64."""
    M, K, N, B = case
    a, w, wp, s = _w4a16_inputs(orc, rng(M * K + N), M, K, N, B)
    print("case: w4a16 any shape", case, flush=True)
    y, kernel = _run_w4a16(pkg, a, wp, s, K, N, B, prepack=False)
    assert kernel == "mtrt_gemm_w4a16_edge"
    _check_w4a16(orc, y, a, w, s, K, N, B, orc.gemm_w4a16(a, wp, s, K, N, B))


@pytest.mark.parametrize("case", [(200, 131, 8), (136, 257, 17), (128, 130, 32)])
def test_w4a16_any_shape_kernel_dequantises_bit_exactly(pkg, orc, case):
    """One-hot activations read the dequantised weights back unchanged: pins the nibble of every (k, n) for odd and
    even N, the block index of the scale when a group of eight k crosses blocks, and the single f16 rounding."""
    K, N, B = case
    g = rng(K + N)
    w = g.integers(-8, 8, (K, N)).astype(np.int8)
    s = orc.narrow(g.uniform(0.005, 0.02, (K // B, N)).astype(np.float32), orc.F16)
    eye = np.zeros((K, K), np.float32)
    np.fill_diagonal(eye, 1.0)
    wd = (w.astype(np.float16) * np.repeat(s.view(np.float16), B, axis=0)).view(np.uint16)
    y, kernel = _run_w4a16(pkg, orc.narrow(eye, orc.F16), orc.pack_int4(w), s, K, N, B, prepack=False)
    assert kernel == "mtrt_gemm_w4a16_edge"
    assert np.array_equal(bits16(y).reshape(K, N), wd)


def test_w4a16_block_of_32_with_re_laid_weights_present(pkg, orc):
    """A block the tile kernels do not take, with both weight layouts passed: the original nibbles are used."""
    M, K, N, B = 100, 512, 192, 32
    a, w, wp, s = _w4a16_inputs(orc, rng(9), M, K, N, B)
    y, kernel = _run_w4a16(pkg, a, wp, s, K, N, B)
    assert kernel == "mtrt_gemm_w4a16_edge"
    _check_w4a16(orc, y, a, w, s, K, N, B, orc.gemm_w4a16(a, wp, s, K, N, B))


@pytest.mark.parametrize("M", [16, 256, 4096])
def test_c5_w4a16_full_size(pkg, orc, M):
    """BASELINE config 5: K=4096, N=11008, block 128, M in {16, 256, 4096}, seed 5.  The oracle
    evaluates up to 40 rows spread over the tiles; all N columns of those rows are compared."""
    K, N, B = 4096, 11008, 128
    a, w, wp, s = _w4a16_inputs(orc, rng(5), M, K, N, B)
    y, kernel = _run_w4a16(pkg, a, wp, s, K, N, B)
    assert kernel in {16: ("mtrt_gemm_w4a16_strips16",), 256: ("mtrt_gemm_w4a16_t128x128",),
                      4096: ("mtrt_gemm_w4a16_t256x384", "mtrt_gemm_w4a16_t256x256")}[M]
    rows = sorted(set([0, M - 1] + list(range(0, M, max(1, M // 38)))))[:40]
    orc.set_threads(16)
    import torch
    got = y[rows].contiguous()
    ref = np.concatenate([orc.gemm_w4a16(a, wp, s, K, N, B, m0=r, mcount=1) for r in rows])
    orc.set_threads(1)
    _check_w4a16(orc, got, a[rows], w, s, K, N, B, ref)
    if M < 256:
        return
    # Every element of the launch against an independent evaluation: weights dequantised with torch (one f16
    # rounding of the exact product), product in float64 on the GPU, the bound of _check_w4a16.
    dev = y.device
    af = torch.from_numpy(a.view(np.float16).astype(np.float32)).to(dev).double()
    wd = (torch.from_numpy(w.astype(np.float16)).to(dev) *
          torch.from_numpy(s.view(np.float16).copy()).to(dev).repeat_interleave(B, dim=0)).double()
    exact = af @ wd
    noise = kNoise * np.sqrt(K) * (af ** 2).mean(dim=1).sqrt()[:, None] * (wd ** 2).mean(dim=0).sqrt()[None, :]
    ulp = torch.exp2(torch.floor(torch.log2(exact.abs().clamp_min(2.0 ** -14)))) * 2.0 ** -10
    err = (y.double() - exact).abs()
    excess = err - (1e-3 * exact.abs() + ulp + noise)
    assert float(excess.max()) <= 0.0, "whole matrix vs float64: worst excess %g at flat index %d" % (
        float(excess.max()), int(excess.argmax()))
    del af, wd, exact, noise, ulp, err, excess
    # ... and every row of one full band of 256-row tiles (all 43 column panels) against the oracle
    band = list(range(256, 512)) if M >= 512 else list(range(0, 256))
    orc.set_threads(16)
    ref = orc.gemm_w4a16(a, wp, s, K, N, B, m0=band[0], mcount=len(band))
    orc.set_threads(1)
    _check_w4a16(orc, y[band].contiguous(), a[band], w, s, K, N, B, ref)


@pytest.mark.parametrize("shape", [(9, 192, 8209), (20, 320, 12000), (32, 256, 16384), (12, 128, 16400), (3, 256, 9000)])
def test_w4a16_small_m_workgroups_with_two_column_tiles(pkg, orc, shape):
    """Between one and two 32-column tiles per compute unit the small-M kernels run one workgroup per
    compute unit and the first ones take a second tile (M > 8); N = 8209 gives 257 tiles (one workgroup
    with two, the last tile ragged), 16384 exactly two each, 16400 one tile too many for that form."""
    M, K, N = shape
    B = 64
    a, w, wp, s = _w4a16_inputs(orc, rng(M + K + N), M, K, N, B)
    y, kernel = _run_w4a16(pkg, a, wp, s, K, N, B)
    assert kernel == ("mtrt_gemm_w4a16_skinny16" if M <= 16 else "mtrt_gemm_w4a16_skinny")
    orc.set_threads(16)
    ref = orc.gemm_w4a16(a, wp, s, K, N, B)
    orc.set_threads(1)
    _check_w4a16(orc, y, a, w, s, K, N, B, ref)


@pytest.mark.parametrize("shape", [(16, 4096, 11008), (16, 384, 16400), (1, 128, 16), (9, 1280, 4099), (13, 640, 8192 + 48),
                                   (16, 256, 40)])
def test_w4a16_strip_kernel(pkg, orc, shape):
    """M <= 16 with K % 128 == 0 and block % 128 == 0: one workgroup per compute unit owning a strip of 16-column
    tiles over all of K (strip-order weights).  N = 11008 gives 688 tiles = 2 or 3 per workgroup, 16400 gives 1025
    (4 or 5: chunks of 3 + 1 and 3 + 2), 4099 a ragged last tile; K = 384 leaves one wave without a K block,
    K = 1280 gives the waves 2 or 3 blocks (no full group of four: the one-at-a-time tail only)."""
    M, K, N = shape
    B = 128
    a, w, wp, s = _w4a16_inputs(orc, rng(M + K + N), M, K, N, B)
    y, kernel = _run_w4a16(pkg, a, wp, s, K, N, B)
    assert kernel == "mtrt_gemm_w4a16_strips16"
    orc.set_threads(16)
    ref = orc.gemm_w4a16(a, wp, s, K, N, B)
    orc.set_threads(1)
    _check_w4a16(orc, y, a, w, s, K, N, B, ref)


def test_w4a16_narrow_mid_tile_kernel(pkg, orc):
    """128 x 64 tiles: matrices at most 64 columns wide (M = 600, N = 40: ragged in M and N), K = 320 (five slices:
    main loop and tail)."""
    M, K, N, B = 600, 320, 40, 64
    a, w, wp, s = _w4a16_inputs(orc, rng(78), M, K, N, B)
    y, kernel = _run_w4a16(pkg, a, wp, s, K, N, B)
    assert kernel == "mtrt_gemm_w4a16_t128x64"
    rows = sorted(set([0, 1, 127, 128, 255, 256, 511, 512, 598, 599] + list(range(3, M, 41))))
    orc.set_threads(16)
    ref = np.concatenate([orc.gemm_w4a16(a, wp, s, K, N, B, m0=r, mcount=1) for r in rows])
    orc.set_threads(1)
    _check_w4a16(orc, y[rows].contiguous(), a[rows], w, s, K, N, B, ref)


@pytest.mark.parametrize("N,want", [(8000, "mtrt_gemm_w4a16_t256x256"), (16416, "mtrt_gemm_w4a16_t256x384")])
def test_w4a16_big_tile_kernel_ragged_edges(pkg, orc, N, want):
    """The 256-row tile kernels on shapes whose M and N are not multiples of the tile (M = 2000; N = 8000 = 250 column
    tiles of 32: one full round of 256 x 256 tiles on 256 compute units; N = 16416 = 513 column tiles: 256 x 384 tiles
    save a round), K = 256 so the oracle stays cheap."""
    import torch
    M, K, B = 2000, 256, 128
    a, w, wp, s = _w4a16_inputs(orc, rng(77), M, K, N, B)
    y, kernel = _run_w4a16(pkg, a, wp, s, K, N, B)
    if torch.cuda.get_device_properties(0).multi_processor_count == 256:
        assert kernel == want
    assert kernel in ("mtrt_gemm_w4a16_t256x256", "mtrt_gemm_w4a16_t256x384")
    rows = sorted(set([0, 1, 127, 128, 255, 256, 1023, 1791, 1792, 1998, 1999] + list(range(5, M, 97))))
    orc.set_threads(16)
    ref = np.concatenate([orc.gemm_w4a16(a, wp, s, K, N, B, m0=r, mcount=1) for r in rows])
    orc.set_threads(1)
    _check_w4a16(orc, y[rows].contiguous(), a[rows], w, s, K, N, B, ref)


@pytest.mark.parametrize("shape,kernel", [((1536, 4096), "t128x256"), ((600, 8480), "t128x256"), ((2048, 4096), "t128x256"), ((1024, 4096), "t128x128"),
                                          ((768, 11008), "t256x256"), ((1536, 11008), "t256x384"), ((3072, 4096), "t256x256")])
def test_w4a16_tile_choice_and_results_at_mid_m(pkg, orc, shape, kernel):
    """The tile is chosen by the estimated number of rounds of one tile per compute unit: 128 x 128 tiles where the
    larger ones would fill half of the units or spill a few tiles into another round, 128 x 256 and 256 x 384 where
    they save a round.  Sampled rows against the oracle for each choice (the expected choice is that of 256 compute units)."""
    M, N = shape
    K, B = 256, 128
    a, w, wp, s = _w4a16_inputs(orc, rng(M + N), M, K, N, B)
    y, k = _run_w4a16(pkg, a, wp, s, K, N, B)
    import torch
    if torch.cuda.get_device_properties(0).multi_processor_count == 256:
        assert k == "mtrt_gemm_w4a16_" + kernel
    assert k in ("mtrt_gemm_w4a16_t128x128", "mtrt_gemm_w4a16_t128x256", "mtrt_gemm_w4a16_t256x256", "mtrt_gemm_w4a16_t256x384")
    rows = sorted(set([0, 1, 127, 128, 255, 256, M - 2, M - 1] + list(range(7, M, 113))))
    orc.set_threads(16)
    ref = np.concatenate([orc.gemm_w4a16(a, wp, s, K, N, B, m0=r, mcount=1) for r in rows])
    orc.set_threads(1)
    _check_w4a16(orc, y[rows].contiguous(), a[rows], w, s, K, N, B, ref)
