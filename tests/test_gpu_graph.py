"""The cluster entry points under HIP graph capture: a captured dynamic-fp8 pipeline (amax -> scale on
device -> fused quantize + dequantize -> LayerNorm) replays with the results of the eager run, several times,
with eager work and synchronisations between the replays.  Nothing in these entry points allocates, memsets
or synchronises, so they can be recorded; the amax reduction cleans its own scratch at the end of each launch."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_captured_pipeline_replays_like_eager(pkg):
    import torch
    L = pkg.lib()
    rows, d = 512, 2048
    n = rows * d
    torch.manual_seed(11)
    x = torch.randn(rows, d, device="cuda").to(torch.bfloat16)
    gamma = (torch.rand(d, device="cuda") + 0.5).to(torch.bfloat16)
    beta = (torch.randn(d, device="cuda") * 0.1).to(torch.bfloat16)
    amax_scale = torch.zeros(2, device="cuda")
    q = torch.zeros(n, dtype=torch.uint8, device="cuda")
    y = torch.zeros(rows, d, dtype=torch.bfloat16, device="cuda")
    z = torch.zeros(rows, d, dtype=torch.bfloat16, device="cuda")
    vp = ctypes.c_void_p

    def pipeline(stream):
        s = vp(stream)
        pkg.check(L.mtrt_hip_amax(s, vp(x.data_ptr()), pkg.BF16, n, ctypes.c_float(448.0), vp(amax_scale.data_ptr()),
                                  vp(amax_scale.data_ptr() + 4)))
        pkg.check(L.mtrt_hip_quantize_dequantize(s, vp(x.data_ptr()), pkg.BF16, vp(q.data_ptr()), pkg.F8E4M3FN, vp(y.data_ptr()),
                                                 vp(amax_scale.data_ptr() + 4), pkg.SCALE_UNIFORM, rows, d, 1, 0))
        pkg.check(L.mtrt_hip_layernorm(s, vp(y.data_ptr()), vp(gamma.data_ptr()), vp(beta.data_ptr()), vp(z.data_ptr()),
                                       pkg.BF16, rows, d, ctypes.c_float(1e-5)))

    def snapshot():
        torch.cuda.synchronize()
        return amax_scale.clone(), q.clone(), y.clone(), z.clone()

    def clear():
        for t in (amax_scale, q, y, z):
            t.zero_()

    pipeline(torch.cuda.current_stream().cuda_stream)           # eager: also brings the device state up before capture
    want = snapshot()
    assert float(want[0][0]) == float(x.float().abs().max())

    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        pipeline(side.cuda_stream)                              # the side stream's reduction scratch exists before capture
        torch.cuda.synchronize()
        graph.capture_begin()
        pipeline(side.cuda_stream)
        graph.capture_end()
    for replay in range(4):
        clear()
        torch.cuda.synchronize()
        graph.replay()
        got = snapshot()
        for g, w, name in zip(got, want, ("amax/scale", "codes", "dequantized", "layernorm")):
            assert torch.equal(g.view(torch.uint8), w.view(torch.uint8)), "replay %d: %s differ from the eager run" % (replay, name)
        # eager work between the replays, on new data, must not disturb the next replay
        x2 = torch.randn(64, 256, device="cuda").to(torch.bfloat16)
        a2, _ = pkg.amax(x2, 448.0)
        assert float(a2) == float(x2.float().abs().max())


def test_captured_one_launch_dynamic_quantization_replays_like_eager(pkg):
    """The one-launch amax + quantize + dequantize kernel (workgroups that wait for each other, a scratch block that
    restores itself) recorded into a graph: every replay gives the eager bits, also after eager launches in between."""
    import torch
    L = pkg.lib()
    torch.manual_seed(12)
    x = torch.randn(1024, 4096, device="cuda")
    n = x.numel()
    out = torch.zeros(2, device="cuda")
    q = torch.zeros(n, dtype=torch.int8, device="cuda")
    y = torch.zeros_like(x)
    vp = ctypes.c_void_p

    def run(stream):
        pkg.check(L.mtrt_hip_dynamic_quantize_dequantize(vp(stream), vp(x.data_ptr()), pkg.F32, vp(q.data_ptr()), pkg.I8,
                                                         vp(y.data_ptr()), n, ctypes.c_float(127.0), vp(out.data_ptr()),
                                                         vp(out.data_ptr() + 4), 0))

    run(torch.cuda.current_stream().cuda_stream)
    assert pkg.last_kernel() == "mtrt_dynqdq_f32_i8_v4"
    torch.cuda.synchronize()
    want = (out.clone(), q.clone(), y.clone())
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        run(side.cuda_stream)
        torch.cuda.synchronize()
        graph.capture_begin()
        run(side.cuda_stream)
        graph.capture_end()
    for replay in range(4):
        for t in (out, q, y):
            t.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for g, w, name in zip((out, q, y), want, ("amax/scale", "codes", "dequantized")):
            assert torch.equal(g.view(torch.uint8), w.view(torch.uint8)), "replay %d: %s differ from the eager run" % (replay, name)
        x2 = torch.randn(300, 1024, device="cuda")
        q2, y2, a2, s2 = pkg.dynamic_quantize_dequantize(x2, pkg.I8, 127.0)
        assert float(a2) == float(x2.abs().max())
