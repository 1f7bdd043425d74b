"""The allocation-free amax entry point (mtrt_hip_amax_no_alloc) against the entry point it is a variant of
(mtrt_hip_amax), bit for bit, through the C ABI: two calls in a row on one stream, the second on a smaller
input, for each input type; the same pair recorded into a HIP graph and replayed on new data; then the argument checks.  Both entry points are also compared with the oracle so
that a shared mistake cannot hide."""
import numpy as np
import pytest

from helpers import rng

pytestmark = pytest.mark.gpu


def _call(pkg, fn, x, n, qmax, out):
    import torch
    pkg.check(fn(torch.cuda.current_stream().cuda_stream, x.data_ptr(), pkg.float_dtype_of(x), n, float(qmax),
                 out.data_ptr(), out.data_ptr() + 4))


def _call_on(pkg, fn, stream, x, n, qmax, out):
    pkg.check(fn(stream, x.data_ptr(), pkg.float_dtype_of(x), n, float(qmax), out.data_ptr(), out.data_ptr() + 4))


@pytest.mark.parametrize("dtype_name", ["f32", "bf16", "f16"])
def test_no_alloc_amax_equals_amax_two_calls_in_a_row(pkg, orc, dtype_name):
    import torch
    L = pkg.lib()
    pkg.check(L.mtrt_hip_init())
    dev = torch.device("cuda:0")
    tdt = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[dtype_name]
    odt = {"f32": orc.F32, "bf16": orc.BF16, "f16": orc.F16}[dtype_name]
    g = rng(77)
    big = torch.from_numpy(g.standard_normal(3 * 1024 * 1024 + 37, dtype=np.float32)).to(dev).to(tdt)
    small = torch.from_numpy((g.standard_normal(4099, dtype=np.float32) * 0.01)).to(dev).to(tdt)
    for x, qmax in ((big, 127.0), (small, 448.0)):      # second call: smaller input, smaller values
        print("no_alloc amax", dtype_name, x.numel(), flush=True)
        ref = torch.full((2,), -1.0, dtype=torch.float32, device=dev)
        got = torch.full((2,), -2.0, dtype=torch.float32, device=dev)
        _call(pkg, L.mtrt_hip_amax, x, x.numel(), qmax, ref)
        _call(pkg, L.mtrt_hip_amax_no_alloc, x, x.numel(), qmax, got)
        torch.cuda.synchronize()
        assert got.cpu().numpy().tobytes() == ref.cpu().numpy().tobytes(), (got, ref)
        storage = x.cpu().numpy().ravel() if odt == orc.F32 else x.view(torch.int16).cpu().numpy().view(np.uint16).ravel()
        amax_ref = orc.amax(storage, odt)
        assert np.float32(got[0].item()).tobytes() == amax_ref.tobytes()
        assert np.float32(got[1].item()).tobytes() == orc.scale_from_amax(amax_ref, qmax).tobytes()


def test_no_alloc_amax_under_graph_capture(pkg, orc):
    """The clear + reduction pair recorded into a graph (the caller this entry point is for): two replays on different
    data, with eager work and synchronisations in between, each compared bit for bit with mtrt_hip_amax."""
    import torch
    L = pkg.lib()
    pkg.check(L.mtrt_hip_init())
    g = rng(78)
    n = 1024 * 1024 + 24
    x = torch.zeros(n, device="cuda:0")
    got = torch.zeros(2, device="cuda:0")
    ref = torch.zeros(2, device="cuda:0")
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        _call_on(pkg, L.mtrt_hip_amax_no_alloc, side.cuda_stream, x, n, 127.0, got)     # once eagerly on the capture stream
        torch.cuda.synchronize()
        graph.capture_begin()
        _call_on(pkg, L.mtrt_hip_amax_no_alloc, side.cuda_stream, x, n, 127.0, got)
        graph.capture_end()
    for replay, scale in enumerate((1.0, 0.03)):
        print("no_alloc amax graph replay", replay, flush=True)
        x.copy_(torch.from_numpy(g.standard_normal(n, dtype=np.float32) * np.float32(scale)))
        got.fill_(-2.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        _call(pkg, L.mtrt_hip_amax, x, n, 127.0, ref)
        torch.cuda.synchronize()
        assert got.cpu().numpy().tobytes() == ref.cpu().numpy().tobytes(), (replay, got, ref)
        assert np.float32(got[0].item()).tobytes() == orc.amax(x.cpu().numpy(), orc.F32).tobytes()


def test_no_alloc_amax_rejects_what_it_cannot_take(pkg):
    import torch
    L = pkg.lib()
    pkg.check(L.mtrt_hip_init())
    x = torch.zeros(16, device="cuda:0")
    out = torch.zeros(2, device="cuda:0")
    s = torch.cuda.current_stream().cuda_stream
    too_many = (1 << 36) + 1
    assert L.mtrt_hip_amax_no_alloc(s, x.data_ptr(), pkg.F32, too_many, 127.0, out.data_ptr(), out.data_ptr() + 4) == 1
    assert b"exceed" in L.mtrt_hip_last_error()
    assert L.mtrt_hip_amax_no_alloc(s, x.data_ptr(), pkg.I8, 16, 127.0, out.data_ptr(), out.data_ptr() + 4) == 1
    assert L.mtrt_hip_amax_no_alloc(s, None, pkg.F32, 16, 127.0, out.data_ptr(), out.data_ptr() + 4) == 1
    # empty input: amax 0, like the existing entry point
    pkg.check(L.mtrt_hip_amax_no_alloc(s, x.data_ptr(), pkg.F32, 0, 127.0, out.data_ptr(), out.data_ptr() + 4))
    torch.cuda.synchronize()
    assert out[0].item() == 0.0
