#!/usr/bin/env python3
"""Benchmark of the quantization / generated-kernel hot path on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|c1|c2a|c2b|c3|c4|c5]

A STEP is one pass of the hot path over one batch of seeded synthetic input: the
programs of BASELINE.json's configs run back to back through the C ABI
(libmtrt_hip.so) on tensors already resident in HBM:
    C1  amax + quantize->dequantize, ONE launch   f32 [1024,4096] -> i8    (per-tensor, amax/127)
    C2a LayerNorm                           bf16 [8192,4096]
    C2b softmax                             f16 [4096,4096]
    C3  amax + fused quantize->dequantize   bf16 [16384,8192] -> f8E4M3FN  (amax/448)
    C4  W8A8 GEMM + dequantize epilogue     M=2048 K=4096 N=11008          (weights re-laid once, untimed)
    C5  W4A16 block-wise GEMM               M in {16,256,4096} K=4096 N=11008 block 128
The metric is BASELINE.json's: achieved HBM GB/s (memory-bound kernels) and MFMA
TOPS (GEMMs) as a percentage of MI355X peak.  For a step that mixes both, `value`
is the time-weighted percentage: 100 * (sum over kernels of the time the kernel
would take at its roofline peak, on its ALGORITHMIC bytes or ops) / (measured time
of the step).  Peaks: HBM 8 TB/s, int8 MFMA 5 POP/s, f16 MFMA 2.5 PFLOP/s.
Every kernel also gets its own line under "workloads" (achieved, peak, fraction),
timed with HIP events on the launch stream over rotating buffers whose combined
footprint exceeds the 256 MiB Infinity Cache, so cache hits do not count as HBM; the
figure is the MEDIAN over ten batches of launches.
Before the W warm-up steps the step runs `--settle-steps` more times, untimed (default 100, about 70 ms): the
board's power management takes 10-15 ms of sustained load after an idle period to settle, and the set-up leaves the GPU
idle; "settle_steps" in the line says how many were run.
"roofline" repeats the entry of the kernel with the largest share of the step.
"mfma_sustained" is the matrix-core rate a loop of nothing but MFMAs reaches on the bench's
own operand data (the published dense peaks hold for idle data only: the clock drops under
the board's power limit); GEMM entries carry "frac_of_sustained" beside "frac".
"hbm_sustained" is the matching yardstick for the memory-bound kernels: a stream that is only read, one that is only
written and a plain copy, over 1 GiB each; HBM entries carry "frac_of_sustained" against the yardstick with their
access mix ("sustained_mix"), and "same_size_yardstick_us": the time of ONE launch of that yardstick moving as many
bytes as the workload does (the 1 GiB rate is out of reach of any launch of a few tens of MB).
"library_yardsticks" are the vendor library's plain GEMMs (torch.matmul f16, torch._int_mm) at the same shapes,
timed the same way; they are not part of the step.
"cpu_baseline" times the CPU oracle (a C++ restatement of the reference's host
lowering, NOT the reference binary) on a bounded sample, single-threaded like the
reference interpreter, and extrapolates linearly to the step; "cpu_baseline_all_cores"
is the same sample with the oracle's OpenMP loops on every host core.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

HBM_PEAK = 8000.0       # GB/s
INT8_PEAK = 5000.0      # TOP/s dense
F16_PEAK = 2500.0       # TFLOP/s dense
CACHE_BYTES = 512 << 20  # rotate buffers over at least this much


def build_workloads(pkg, torch, which):
    """Returns a list of kernel descriptors.  Each has: name (kernel symbol or short label),
    config, bound ('hbm'|'mfma'), work (algorithmic bytes or ops per launch), peak, unit,
    make(slot) -> zero-argument callable that enqueues one launch on buffer set `slot`, nslots."""
    L = pkg.lib()
    dev = torch.device("cuda:0")
    out = []

    def stream():
        return torch.cuda.current_stream().cuda_stream

    def gen(shape, dtype, seed, scale=1.0):
        g = torch.Generator(device=dev)
        g.manual_seed(seed)
        return (torch.randn(shape, generator=g, device=dev, dtype=torch.float32) * scale).to(dtype)

    def slots_for(bytes_per_set):
        return max(2, int(np.ceil(CACHE_BYTES / bytes_per_set)))

    if which in ("all", "c1"):
        n = 1024 * 4096
        ns = slots_for(n * 9)
        x1 = [gen((1024, 4096), torch.float32, 1 + i) for i in range(ns)]
        q1 = [torch.empty(n, dtype=torch.int8, device=dev) for _ in range(ns)]
        y1 = [torch.empty_like(x) for x in x1]
        s1 = [torch.empty(2, dtype=torch.float32, device=dev) for _ in range(ns)]

        def dynq(i, xs=x1, qs=q1, ys=y1, sc=s1, n=n):
            a = (xs[i].data_ptr(), pkg.F32, qs[i].data_ptr(), pkg.I8, ys[i].data_ptr(), n, 127.0, sc[i].data_ptr(),
                 sc[i].data_ptr() + 4, 0)
            return lambda: pkg.check(L.mtrt_hip_dynamic_quantize_dequantize(stream(), *a))
        # one launch: x read once (kept in registers across the reduction), q and y written: 9 bytes per element
        out.append(dict(name="mtrt_dynqdq_f32_i8_v4", config="C1", bound="hbm", work=9.0 * n, nslots=ns, make=dynq,
                        keep=(x1, q1, y1, s1)))

    if which in ("all", "c2a"):
        rows, d = 8192, 4096
        ns = slots_for(rows * d * 4)
        xs = [gen((rows, d), torch.bfloat16, 20 + i) for i in range(ns)]
        ys = [torch.empty_like(x) for x in xs]
        gg = torch.Generator(device=dev)
        gg.manual_seed(19)
        gamma = (torch.rand(d, generator=gg, device=dev) + 0.5).to(torch.bfloat16)
        beta = (torch.randn(d, generator=gg, device=dev) * 0.1).to(torch.bfloat16)

        def ln(i, xs=xs, ys=ys, rows=rows, d=d, gamma=gamma, beta=beta):
            a = (xs[i].data_ptr(), gamma.data_ptr(), beta.data_ptr(), ys[i].data_ptr(), pkg.BF16, rows, d, 1e-5)
            return lambda: pkg.check(L.mtrt_hip_layernorm(stream(), *a))
        # the library picks the 64-register form of the kernel when eight waves per SIMD hold every row at once
        simds = 4 * torch.cuda.get_device_properties(0).multi_processor_count
        ln_name = "mtrt_layernorm_bf16_v8" + ("r" if 5 * simds < rows <= 8 * simds else "")
        out.append(dict(name=ln_name, config="C2a", bound="hbm", work=4.0 * rows * d + 4.0 * d,
                        nslots=ns, make=ln, keep=(xs, ys, gamma, beta)))

    if which in ("all", "c2b"):
        rows, d = 4096, 4096
        ns = slots_for(rows * d * 4)
        xs = [gen((rows, d), torch.float16, 40 + i, 2.0) for i in range(ns)]
        ys = [torch.empty_like(x) for x in xs]

        def sm(i, xs=xs, ys=ys, rows=rows, d=d):
            a = (xs[i].data_ptr(), ys[i].data_ptr(), pkg.F16, rows, d)
            return lambda: pkg.check(L.mtrt_hip_softmax(stream(), *a))
        out.append(dict(name="mtrt_softmax_f16_v8", config="C2b", bound="hbm", work=4.0 * rows * d, nslots=ns, make=sm,
                        keep=(xs, ys)))

    if which in ("all", "c3"):
        rows, cols = 16384, 8192
        n = rows * cols
        ns = 2
        xs = []
        for i in range(ns):
            x = gen((rows, cols), torch.float32, 60 + i, float(np.sqrt(2.0)))
            g = torch.Generator(device=dev)
            g.manual_seed(600 + i)
            x[torch.rand((rows, cols), generator=g, device=dev) < 0.001] *= 50.0
            xs.append(x.to(torch.bfloat16))
            del x
        qs = [torch.empty(n, dtype=torch.uint8, device=dev) for _ in range(ns)]
        ys = [torch.empty_like(x) for x in xs]
        sc = [torch.empty(2, dtype=torch.float32, device=dev) for _ in range(ns)]

        def amax(i, xs=xs, sc=sc, n=n):
            a = (xs[i].data_ptr(), pkg.BF16, n, 448.0, sc[i].data_ptr(), sc[i].data_ptr() + 4)
            return lambda: pkg.check(L.mtrt_hip_amax(stream(), *a))

        def qdq(i, xs=xs, qs=qs, ys=ys, sc=sc, rows=rows, cols=cols):
            a = (xs[i].data_ptr(), pkg.BF16, qs[i].data_ptr(), pkg.F8E4M3FN, ys[i].data_ptr(), sc[i].data_ptr() + 4,
                 pkg.SCALE_UNIFORM, rows, cols, 1, 0)
            return lambda: pkg.check(L.mtrt_hip_quantize_dequantize(stream(), *a))
        out.append(dict(name="mtrt_amax_bf16", config="C3", bound="hbm", work=2.0 * n, nslots=ns, make=amax, keep=(xs, sc),
                        mix="read"))
        out.append(dict(name="mtrt_qdq_uniform_bf16_f8", config="C3", bound="hbm", work=5.0 * n, nslots=ns, make=qdq,
                        keep=(qs, ys)))

    if which == "nvfp4":
        # Not a BASELINE config (and not part of "all"): the NVFP4 block quantize / dequantize pair on the
        # tensor of config 3, for its own roofline line.
        rows, cols = 16384, 8192
        n = rows * cols
        ns = 2
        xs = [gen((rows, cols), torch.float32, 80 + i, float(np.sqrt(2.0))).to(torch.bfloat16) for i in range(ns)]
        qs = [torch.empty(n // 2, dtype=torch.uint8, device=dev) for _ in range(ns)]
        ss = [torch.empty(n // 16, dtype=torch.uint8, device=dev) for _ in range(ns)]
        ys = [torch.empty_like(x) for x in xs]
        am = [x.float().abs().max().reshape(1).contiguous() for x in xs]

        def nvq(i, xs=xs, qs=qs, ss=ss, am=am, rows=rows, cols=cols):
            a = (xs[i].data_ptr(), pkg.BF16, qs[i].data_ptr(), ss[i].data_ptr(), am[i].data_ptr(), rows, cols, 1)
            return lambda: pkg.check(L.mtrt_hip_nvfp4_quantize(stream(), *a))

        def nvdq(i, qs=qs, ss=ss, am=am, ys=ys, rows=rows, cols=cols):
            a = (qs[i].data_ptr(), ss[i].data_ptr(), am[i].data_ptr(), ys[i].data_ptr(), pkg.BF16, rows, cols, 1)
            return lambda: pkg.check(L.mtrt_hip_nvfp4_dequantize(stream(), *a))
        out.append(dict(name="mtrt_nvfp4_q_bf16", config="NVFP4 (C3 tensor)", bound="hbm", work=(2.0 + 0.5 + 1.0 / 16) * n,
                        nslots=ns, make=nvq, keep=(xs, qs, ss, am)))
        out.append(dict(name="mtrt_nvfp4_dq_bf16", config="NVFP4 (C3 tensor)", bound="hbm", work=(2.0 + 0.5 + 1.0 / 16) * n,
                        nslots=ns, make=nvdq, keep=(ys,)))

    if which in ("all", "c4"):
        M, K, N = 2048, 4096, 11008
        ns = slots_for(M * K + K * N + 2 * M * N)
        g = torch.Generator(device=dev)
        g.manual_seed(4)

        def q8(shape):
            return torch.clamp(torch.round(torch.randn(shape, generator=g, device=dev) * 40.0), -128, 127).to(torch.int8)
        a4 = [q8((M, K)) for _ in range(ns)]
        w4 = [pkg.gemm_w8a8_prepack_fragments(q8((K, N))) for _ in range(ns)]   # weights are constants: re-laid once, untimed
        as4 = (torch.rand(M, generator=g, device=dev) * 0.015 + 0.005)
        ws4 = (torch.rand(N, generator=g, device=dev) * 0.015 + 0.005)
        y4 = [torch.empty((M, N), dtype=torch.float16, device=dev) for _ in range(ns)]

        def gemm8(i, a4=a4, w4=w4, y4=y4, as4=as4, ws4=ws4, M=M, K=K, N=N):
            a = (a4[i].data_ptr(), w4[i].data_ptr(), as4.data_ptr(), ws4.data_ptr(), y4[i].data_ptr(), M, K, N)
            return lambda: pkg.check(L.mtrt_hip_gemm_w8a8_fragments(stream(), *a))
        # the same launch on all-zero operands: same instructions and memory traffic, no switching activity in the
        # matrix cores; the difference to the timed launch is what the board's power limit costs on this data
        az = torch.zeros((M, K), dtype=torch.int8, device=dev)
        wz = torch.zeros_like(w4[0])

        def gemm8_zero(i, az=az, wz=wz, y4=y4, as4=as4, ws4=ws4, M=M, K=K, N=N):
            a = (az.data_ptr(), wz.data_ptr(), as4.data_ptr(), ws4.data_ptr(), y4[i].data_ptr(), M, K, N)
            return lambda: pkg.check(L.mtrt_hip_gemm_w8a8_fragments(stream(), *a))
        out.append(dict(name="mtrt_gemm_w8a8_frag_t256x384", dispatched=True, config="C4", bound="mfma", work=2.0 * M * K * N, peak=INT8_PEAK,
                        unit="TOP/s", nslots=ns, make=gemm8, keep=(a4, w4, y4, as4, ws4, az, wz),
                        probe=("mtrt_mfma_probe_i8", w4[0], 65536.0), zero_operands=gemm8_zero))

    if which in ("all", "c5"):
        K, N, B = 4096, 11008, 128
        g = torch.Generator(device=dev)
        g.manual_seed(5)
        for M, kname in ((16, "mtrt_gemm_w4a16_strips16"), (256, "mtrt_gemm_w4a16_t128x128"), (4096, "mtrt_gemm_w4a16_t256x256")):
            nbytes = K * N // 2 + (K // B) * N * 2 + M * K * 2 + M * N * 2
            ns = min(slots_for(nbytes), 24)
            a5 = [torch.randn((M, K), generator=g, device=dev).half() for _ in range(ns)]
            w5 = [pkg.gemm_w4a16_prepack(torch.randint(0, 256, (K * N // 2,), generator=g, device=dev, dtype=torch.uint8), K, N)
                  for _ in range(ns)]                                      # re-laid once, untimed
            s5 = [(torch.rand((K // B, N), generator=g, device=dev) * 0.015 + 0.005).half() for _ in range(ns)]
            y5 = [torch.empty((M, N), dtype=torch.float16, device=dev) for _ in range(ns)]

            def gemm4(i, a5=a5, w5=w5, s5=s5, y5=y5, M=M):
                a = (a5[i].data_ptr(), None, w5[i].data_ptr(), s5[i].data_ptr(), y5[i].data_ptr(), M, K, N, B)
                return lambda: pkg.check(L.mtrt_hip_gemm_w4a16(stream(), *a))
            if M == 16:      # arithmetic intensity ~61 FLOP/B: bound by reading the weights once
                out.append(dict(name=kname, config="C5 M=16", bound="hbm", work=float(nbytes), nslots=ns, make=gemm4,
                                keep=(a5, w5, s5, y5), mix="read"))
            else:
                zero = None
                if M == 4096:    # the same launch with zero activations and zero weights (nibble 8 is the value 0)
                    az5 = torch.zeros((M, K), dtype=torch.float16, device=dev)
                    wz5 = torch.full_like(w5[0], 0x88)

                    def zero(i, az5=az5, wz5=wz5, s5=s5, y5=y5, M=M):
                        a = (az5.data_ptr(), None, wz5.data_ptr(), s5[i].data_ptr(), y5[i].data_ptr(), M, K, N, B)
                        return lambda: pkg.check(L.mtrt_hip_gemm_w4a16(stream(), *a))
                out.append(dict(name=kname, dispatched=True, config="C5 M=%d" % M, bound="mfma", work=2.0 * M * K * N, peak=F16_PEAK,
                                unit="TFLOP/s", nslots=ns, make=gemm4, keep=(a5, w5, s5, y5),
                                probe=("mtrt_mfma_probe_f16", a5[0], 32768.0) if M == 4096 else None, zero_operands=zero))

    for w in out:
        w["peak"] = HBM_PEAK if w["bound"] == "hbm" else w["peak"]
        w["unit"] = "GB/s" if w["bound"] == "hbm" else w["unit"]
    return out


_YARDSTICKS = []


def yardstick_module(pkg):
    """The code object with the measurement yardsticks (plain copy, matrix-core-only loop); they are not part of
    the library's built-in module."""
    if not _YARDSTICKS:
        path = pkg.FIXTURE_MODULE_PATH.encode()
        _YARDSTICKS.append(pkg.lib().mtrt_cuda_module_load_from_ptx_file(path, len(path)))
    return _YARDSTICKS[0]


def calibration_copy(pkg, torch):
    """One launch of the plain copy kernel over 128 MiB (reads 128 MiB, writes 128 MiB): the
    yardstick that hardware byte counters of a profiled run are scaled by."""
    import ctypes
    L = pkg.lib()
    nbytes = 128 << 20
    src = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    dst = torch.empty_like(src)
    src.fill_(1)
    name = b"mtrt_copy_b128"
    fn = L.mtrt_cuda_module_get_function(yardstick_module(pkg), name, len(name))
    vals = (ctypes.c_void_p(src.data_ptr()), ctypes.c_void_p(dst.data_ptr()), ctypes.c_int64(nbytes // 16))
    args = (ctypes.c_void_p * 3)(*[ctypes.cast(ctypes.pointer(v), ctypes.c_void_p) for v in vals])
    nvec = nbytes // 16
    L.mtrt_cuda_launch_kernel(fn, nvec // 256, 1, 1, 256, 1, 1, 0, torch.cuda.current_stream().cuda_stream, args)
    torch.cuda.synchronize()


def mfma_sustained(pkg, torch, kernel, operand, ops_per_mfma):
    """Rate (T ops/s) of the matrix-core yardstick kernel on `operand`'s bytes: 16 independent
    MFMAs per round and wave, one wave per SIMD, no memory traffic in the loop."""
    import ctypes
    L = pkg.lib()
    dev = L.mtrt_cuda_get_current_device()
    units = torch.cuda.get_device_properties(0).multi_processor_count
    ksteps = 2048
    out = torch.empty(units * 256, dtype=torch.int32, device="cuda")
    assert operand.numel() * operand.element_size() >= (1 << 24)
    name = kernel.encode()
    fn = L.mtrt_cuda_module_get_function(yardstick_module(pkg), name, len(name))
    vals = (ctypes.c_void_p(operand.data_ptr()), ctypes.c_void_p(out.data_ptr()), ctypes.c_int32(ksteps))
    args = (ctypes.c_void_p * 3)(*[ctypes.cast(ctypes.pointer(v), ctypes.c_void_p) for v in vals])
    s = torch.cuda.current_stream().cuda_stream

    def launch():
        L.mtrt_cuda_launch_kernel(fn, units, 1, 1, 256, 1, 1, 0, s, args)
    for _ in range(2):
        launch()
    e0, e1 = L.mtrt_cuda_event_create(dev), L.mtrt_cuda_event_create(dev)
    L.mtrt_cuda_stream_record_event(s, e0)
    reps = 5
    for _ in range(reps):
        launch()
    L.mtrt_cuda_stream_record_event(s, e1)
    L.mtrt_cuda_event_sync(e1)
    us = L.mtrt_cuda_event_elapsed_msec(e0, e1) * 1e3 / reps
    L.mtrt_cuda_event_release(e0)
    L.mtrt_cuda_event_release(e1)
    return ksteps * 16.0 * units * 4 * ops_per_mfma / us / 1e6


def hbm_sustained(pkg, torch, sizes=(), reps=200, nbytes=1 << 30):
    """What the memory system sustains on this box for the three access mixes of the memory-bound clusters, each as
    one launch of a yardstick kernel over `nbytes` (one 128-bit access per lane, one-shot grid, buffers far larger than
    the 256 MiB Infinity Cache): {"read": GB/s of a stream that is only read, "write": only written, "copy": bytes
    read + bytes written of a plain copy}.  Timed like the clusters: HIP events on the launch stream, median of ten."""
    import ctypes
    L = pkg.lib()
    dev = L.mtrt_cuda_get_current_device()
    s = torch.cuda.current_stream().cuda_stream
    src = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    dst = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    sink = torch.zeros(4, dtype=torch.int32, device="cuda")
    src.fill_(1)
    dst.fill_(2)
    nvec = nbytes // 16
    grid = nvec // 256

    def launcher(name, vals):
        fn = L.mtrt_cuda_module_get_function(yardstick_module(pkg), name, len(name))
        args = (ctypes.c_void_p * len(vals))(*[ctypes.cast(ctypes.pointer(v), ctypes.c_void_p) for v in vals])
        return lambda keep=(vals, args): L.mtrt_cuda_launch_kernel(fn, grid, 1, 1, 256, 1, 1, 0, s, args)
    kinds = (
        ("read", launcher(b"mtrt_read_b128", (ctypes.c_void_p(src.data_ptr()), ctypes.c_void_p(sink.data_ptr()),
                                              ctypes.c_int64(nvec), ctypes.c_uint32(0))), nbytes),
        ("write", launcher(b"mtrt_fill_b128", (ctypes.c_void_p(dst.data_ptr()), ctypes.c_int64(nvec), ctypes.c_uint32(3))), nbytes),
        ("copy", launcher(b"mtrt_copy_b128", (ctypes.c_void_p(src.data_ptr()), ctypes.c_void_p(dst.data_ptr()),
                                              ctypes.c_int64(nvec))), 2 * nbytes),
    )
    out = {}
    for kind, launch, moved in kinds:
        for _ in range(3):
            launch()
        events = [L.mtrt_cuda_event_create(dev) for _ in range(11)]
        L.mtrt_cuda_stream_record_event(s, events[0])
        for b in range(10):
            launch()
            L.mtrt_cuda_stream_record_event(s, events[b + 1])
        L.mtrt_cuda_event_sync(events[-1])
        us = sorted(L.mtrt_cuda_event_elapsed_msec(events[b], events[b + 1]) * 1e3 for b in range(10))
        for e in events:
            L.mtrt_cuda_event_release(e)
        out[kind] = round(moved / (0.5 * (us[4] + us[5])) / 1e3, 1)
    # The same yardsticks at the SIZE of each memory-bound workload (`sizes`: (key, bytes moved, mix)): one launch
    # moving as many bytes as the workload's algorithmic traffic (a copy: half read, half written), on rotating
    # windows of the 1 GiB buffers, timed like the workloads (batches of back-to-back launches, median).  A launch of
    # a few tens of MB is far from the 1 GiB rate for any kernel: the chip takes microseconds to fill and drain.
    same_size = {}
    for key, moved, mix in sizes:
        per_stream = (int(moved) // (1 if mix == "read" else 2)) // 4096 * 4096
        if per_stream < 4096 or per_stream > nbytes:
            continue
        nv = per_stream // 16
        nslots = max(1, min(48, nbytes // per_stream))
        name = b"mtrt_read_b128" if mix == "read" else b"mtrt_copy_b128"
        fn = L.mtrt_cuda_module_get_function(yardstick_module(pkg), name, len(name))
        calls = []
        for j in range(nslots):
            if mix == "read":
                vals = (ctypes.c_void_p(src.data_ptr() + j * per_stream), ctypes.c_void_p(sink.data_ptr()), ctypes.c_int64(nv), ctypes.c_uint32(0))
            else:
                vals = (ctypes.c_void_p(src.data_ptr() + j * per_stream), ctypes.c_void_p(dst.data_ptr() + j * per_stream), ctypes.c_int64(nv))
            args = (ctypes.c_void_p * len(vals))(*[ctypes.cast(ctypes.pointer(v), ctypes.c_void_p) for v in vals])
            calls.append(lambda keep=(vals, args), args=args, fn=fn, g=nv // 256: L.mtrt_cuda_launch_kernel(fn, g, 1, 1, 256, 1, 1, 0, s, args))
        us = time_kernel(pkg, torch, dict(make=lambda i, calls=calls: calls[i], nslots=nslots), reps)
        same_size[key] = round(us, 2)
    assert int(sink[0]) == 0
    del src, dst
    return out, same_size


def kernel_sources_digest():
    """sha256 over the device sources (csrc/kernels/*, in name order): what a counter profile must have been taken
    with for its per-kernel figures to describe the kernels that run now."""
    import hashlib
    kdir = os.path.join(ROOT, "tensorrt-incubator_amd", "csrc", "kernels")
    h = hashlib.sha256()
    for name in sorted(os.listdir(kdir)):
        if name.endswith((".hip", ".hpp")):
            h.update(name.encode() + b"\0")
            h.update(open(os.path.join(kdir, name), "rb").read())
    return h.hexdigest()


def traffic_from_profile(kernel):
    """(HBM bytes per launch of `kernel`, where the figure comes from).  The figure is the one measured by the
    committed counter profile (profiles/hbm_traffic_bench_suite.md, table rows `| kernel | fetch | write | total |`);
    it is None when the profile names other kernel sources than the ones in the tree (line `kernel sources sha256:
    ...`), i.e. when it was taken before a kernel changed."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic_bench_suite.md")
    where = "profiles/hbm_traffic_bench_suite.md (rocprofv3 --pmc run of this command; not measured in this run)"
    if not os.path.exists(path):
        return None, "no counter profile in the tree"
    value, digest = None, None
    for line in open(path):
        if line.startswith("kernel sources sha256:"):
            digest = line.split(":", 1)[1].strip()
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if len(cells) >= 4 and cells[0] == kernel:
            try:
                value = float(cells[3])
            except ValueError:
                value = None
    if digest != kernel_sources_digest():
        return None, "profiles/hbm_traffic_bench_suite.md was taken with other kernel sources than the tree's: not used"
    return value, where


def time_kernel(pkg, torch, w, reps):
    """Launch duration in microseconds: HIP events on the launch stream around batches of back-to-back launches
    (`reps` launches in ten batches), the MEDIAN of the batch averages."""
    L = pkg.lib()
    dev = L.mtrt_cuda_get_current_device()
    calls = [w["make"](i) for i in range(w["nslots"])]
    s = torch.cuda.current_stream().cuda_stream
    for c in calls:
        c()
    batches = 10 if reps >= 20 else 1
    per = max(1, reps // batches)
    events = [L.mtrt_cuda_event_create(dev) for _ in range(batches + 1)]
    L.mtrt_cuda_stream_sync(s)
    L.mtrt_cuda_stream_record_event(s, events[0])
    r = 0
    for b in range(batches):
        for _ in range(per):
            calls[r % len(calls)]()
            r += 1
        L.mtrt_cuda_stream_record_event(s, events[b + 1])
    L.mtrt_cuda_event_sync(events[-1])
    us = sorted(L.mtrt_cuda_event_elapsed_msec(events[b], events[b + 1]) * 1e3 / per for b in range(batches))
    for e in events:
        L.mtrt_cuda_event_release(e)
    return us[len(us) // 2] if batches % 2 else 0.5 * (us[batches // 2 - 1] + us[batches // 2])


def cache_variants(pkg, torch, wl, which, reps):
    """The two configurations that fit in the 256 MiB Infinity Cache (C1: 38 MB, C2b: 67 MB), measured two more
    ways beside the rotating-buffer ("cold") figure of the main table: "warm" (one buffer set launched again and
    again, so it stays in the cache) and the same kernels on 16 times the rows (too large for the cache)."""
    L = pkg.lib()
    dev = torch.device("cuda:0")

    def stream():
        return torch.cuda.current_stream().cuda_stream
    out = []
    for w in wl:
        if w["config"] in ("C1", "C2b"):
            us = time_kernel(pkg, torch, dict(w, nslots=1), reps)
            out.append(dict(kernel=w["name"], config=w["config"] + " warm (one buffer set)", us=round(us, 2),
                            achieved=round(w["work"] / us / 1e3, 1), unit="GB/s"))
    if which in ("all", "c1"):
        rows, cols = 16 * 1024, 4096
        n = rows * cols
        gens = [torch.Generator(device=dev) for _ in range(2)]
        for i, gi in enumerate(gens):
            gi.manual_seed(900 + i)
        x = [torch.randn((rows, cols), generator=gi, device=dev) for gi in gens]
        q = [torch.empty(n, dtype=torch.int8, device=dev) for _ in range(2)]
        y = [torch.empty_like(t) for t in x]
        sc = [torch.empty(2, dtype=torch.float32, device=dev) for _ in range(2)]

        def amax(i):
            a = (x[i].data_ptr(), pkg.F32, n, 127.0, sc[i].data_ptr(), sc[i].data_ptr() + 4)
            return lambda: pkg.check(L.mtrt_hip_amax(stream(), *a))

        def qdq(i):
            a = (x[i].data_ptr(), pkg.F32, q[i].data_ptr(), pkg.I8, y[i].data_ptr(), sc[i].data_ptr() + 4, pkg.SCALE_UNIFORM,
                 rows, cols, 1, 0)
            return lambda: pkg.check(L.mtrt_hip_quantize_dequantize(stream(), *a))
        for name, make, work in (("mtrt_amax_f32", amax, 4.0 * n), ("mtrt_qdq_uniform_f32_i8", qdq, 9.0 * n)):
            us = time_kernel(pkg, torch, dict(make=make, nslots=2), max(10, reps // 4))
            out.append(dict(kernel=name, config="C1 x16 rows [16384, 4096]", us=round(us, 2), achieved=round(work / us / 1e3, 1),
                            unit="GB/s"))
        del x, q, y
    if which in ("all", "c2b"):
        rows, d = 16 * 4096, 4096
        gens = [torch.Generator(device=dev) for _ in range(2)]
        for i, gi in enumerate(gens):
            gi.manual_seed(940 + i)
        x = [(torch.randn((rows, d), generator=gi, device=dev) * 2.0).half() for gi in gens]
        y = [torch.empty_like(t) for t in x]

        def sm(i):
            a = (x[i].data_ptr(), y[i].data_ptr(), pkg.F16, rows, d)
            return lambda: pkg.check(L.mtrt_hip_softmax(stream(), *a))
        us = time_kernel(pkg, torch, dict(make=sm, nslots=2), max(10, reps // 4))
        out.append(dict(kernel="mtrt_softmax_f16_v8", config="C2b x16 rows [65536, 4096]", us=round(us, 2),
                        achieved=round(4.0 * rows * d / us / 1e3, 1), unit="GB/s"))
    return out


def extra_clusters(pkg, torch, reps):
    """Clusters that are not one of BASELINE.json's configs and not part of the step or of `value`, each with its own
    roofline line: the per-token dynamic quantization that makes C4's int8 activations and a_scale (f16 [2048, 4096]
    -> int8 codes + f32 scales in one launch; x read once, codes written: 3 bytes per element), beside the two
    launches it replaces (per-row amax, then row-scaled quantize: x read twice, 5 bytes per element)."""
    L = pkg.lib()
    dev = torch.device("cuda:0")
    rows, d = 2048, 4096
    ns = max(2, int(np.ceil(CACHE_BYTES / (rows * d * 3))))
    g = torch.Generator(device=dev)
    g.manual_seed(44)
    xs = [(torch.randn((rows, d), generator=g, device=dev) * 3.0).half() for _ in range(ns)]
    qs = [torch.empty((rows, d), dtype=torch.int8, device=dev) for _ in range(ns)]
    sc = [torch.empty((2, rows), dtype=torch.float32, device=dev) for _ in range(ns)]

    def stream():
        return torch.cuda.current_stream().cuda_stream

    def fused(i):
        a = (xs[i].data_ptr(), pkg.F16, qs[i].data_ptr(), pkg.I8, rows, d, 127.0, sc[i][0].data_ptr(), sc[i][1].data_ptr(), 0)
        return lambda: pkg.check(L.mtrt_hip_dynamic_quantize_rows(stream(), *a))

    def two(i):
        a1 = (xs[i].data_ptr(), pkg.F16, pkg.SCALE_ROW, rows, d, rows, 127.0, sc[i][0].data_ptr(), sc[i][1].data_ptr())
        a2 = (xs[i].data_ptr(), pkg.F16, qs[i].data_ptr(), pkg.I8, sc[i][1].data_ptr(), pkg.SCALE_ROW, rows, d, rows, 0)

        def run():
            pkg.check(L.mtrt_hip_amax_scales(stream(), *a1))
            pkg.check(L.mtrt_hip_quantize(stream(), *a2))
        return run
    out = []
    work = 3.0 * rows * d + 8.0 * rows
    for what, make in (("%s (one launch)", fused), ("mtrt_amax_rows_f16 + %s (two launches)", two)):
        us = time_kernel(pkg, torch, dict(make=make, nslots=ns), reps)
        what = what % pkg.last_kernel()
        out.append(dict(kernel=what, config="per-token int8 quantization of C4's activations, f16 [2048, 4096]", bound="hbm",
                        us=round(us, 2), achieved=round(work / us / 1e3, 1), peak=HBM_PEAK, unit="GB/s",
                        frac=round(work / us / 1e3 / HBM_PEAK, 4), work=work))
    return out


def library_yardsticks(torch, which, reps):
    """The vendor library's plain GEMMs at the benchmark's shapes and on the same kind of data, timed the same way
    (torch.matmul on f16 operands: the weights already dequantised, so it does less work than the W4A16 cluster;
    torch._int_mm for int8 x int8 -> int32, without the scale epilogue).  Not part of the step or of `value`: it shows
    what a tuned library kernel reaches on this chip under the same power limit."""
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev)
    g.manual_seed(77)
    out = []

    def timed(fn, n):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        best = None
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(n):
                fn()
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / n
            best = us if best is None else min(best, us)
        return best

    if which in ("all", "c5"):
        K, N, B = 4096, 11008, 128
        w = torch.randint(-8, 8, (K, N), generator=g, device=dev).half()
        sc = (torch.rand((K // B, N), generator=g, device=dev) * 0.015 + 0.005).half()
        wd = (w * sc.repeat_interleave(B, 0)).half()
        wdt = wd.t().contiguous()
        del w, sc
        for M in (16, 256, 4096):
            a = torch.randn((M, K), generator=g, device=dev).half()
            y = torch.empty((M, N), dtype=torch.float16, device=dev)
            n = max(5, reps // (1 if M <= 256 else 4))
            us = min(timed(lambda: torch.matmul(a, wd, out=y), n), timed(lambda: torch.matmul(a, wdt.t(), out=y), n))
            out.append(dict(what="torch.matmul f16 (weights dequantised beforehand), better of [K,N] and [N,K] weights",
                            config="C5 M=%d" % M, us=round(us, 2), achieved=round(2.0 * M * K * N / us / 1e6, 1), unit="TFLOP/s"))
        del wd, wdt
    if which in ("all", "c4") and hasattr(torch, "_int_mm"):
        M, K, N = 2048, 4096, 11008

        def q8(shape):
            return torch.clamp(torch.round(torch.randn(shape, generator=g, device=dev) * 40.0), -128, 127).to(torch.int8)
        a, w = q8((M, K)), q8((K, N))
        wt = w.t().contiguous()
        try:
            us = min(timed(lambda: torch._int_mm(a, w), max(5, reps // 4)), timed(lambda: torch._int_mm(a, wt.t()), max(5, reps // 4)))
            out.append(dict(what="torch._int_mm int8 -> int32 (no scale epilogue, no f16 output), better of [K,N] and [N,K] weights",
                            config="C4", us=round(us, 2), achieved=round(2.0 * M * K * N / us / 1e6, 1), unit="TOP/s"))
        except RuntimeError:
            pass
    return out


def cpu_baseline(which, threads=1):
    """Times the CPU oracle on a bounded sample of each program, with `threads` OpenMP threads (1 = like the
    reference's single-threaded interpreter), and extrapolates linearly to the full configuration; returns
    (seconds per step, description)."""
    orc = entry.load_oracle()
    orc.set_threads(threads)
    g = np.random.Generator(np.random.PCG64(1))
    total = 0.0
    parts = []

    def timed(fn):
        t0 = time.perf_counter()
        fn()
        return time.perf_counter() - t0

    if which in ("all", "c1"):
        x = g.standard_normal((1024, 4096), dtype=np.float32)
        t = timed(lambda: orc.amax(x, orc.F32))
        s = [orc.scale_from_amax(orc.amax(x, orc.F32), 127.0)]
        q = orc.quantize(x, orc.F32, orc.I8, s, orc.SCALE_UNIFORM, 1024, 4096)
        t += timed(lambda: orc.quantize(x, orc.F32, orc.I8, s, orc.SCALE_UNIFORM, 1024, 4096))
        t += timed(lambda: orc.dequantize(q, orc.I8, orc.F32, s, orc.SCALE_UNIFORM, 1024, 4096))
        total += t
        parts.append("C1 full")
    if which in ("all", "c2a"):
        rows = 1024
        x = orc.narrow(g.standard_normal((rows, 4096), dtype=np.float32), orc.BF16)
        gm = orc.narrow(g.uniform(0.5, 1.5, 4096).astype(np.float32), orc.BF16)
        bt = orc.narrow((g.standard_normal(4096) * 0.1).astype(np.float32), orc.BF16)
        total += timed(lambda: orc.layernorm(x, gm, bt, orc.BF16, rows, 4096, 1e-5)) * (8192 / rows)
        parts.append("C2a %d of 8192 rows" % rows)
    if which in ("all", "c2b"):
        rows = 512
        x = orc.narrow(g.standard_normal((rows, 4096), dtype=np.float32) * 2, orc.F16)
        total += timed(lambda: orc.softmax(x, orc.F16, rows, 4096)) * (4096 / rows)
        parts.append("C2b %d of 4096 rows" % rows)
    if which in ("all", "c3"):
        rows = 1024
        x = orc.narrow(g.standard_normal((rows, 8192), dtype=np.float32) * np.float32(1.414), orc.BF16)
        t = timed(lambda: orc.amax(x, orc.BF16))
        s = [orc.scale_from_amax(orc.amax(x, orc.BF16), 448.0)]
        q = orc.quantize(x, orc.BF16, orc.F8E4M3FN, s, orc.SCALE_UNIFORM, rows, 8192)
        t += timed(lambda: orc.quantize(x, orc.BF16, orc.F8E4M3FN, s, orc.SCALE_UNIFORM, rows, 8192))
        t += timed(lambda: orc.dequantize(q, orc.F8E4M3FN, orc.BF16, s, orc.SCALE_UNIFORM, rows, 8192))
        total += t * (16384 / rows)
        parts.append("C3 %d of 16384 rows" % rows)
    if which in ("all", "c4"):
        M, K, N, rows = 2048, 4096, 11008, 8
        a = np.clip(np.rint(g.standard_normal((rows, K)) * 40), -128, 127).astype(np.int8)
        w = np.clip(np.rint(g.standard_normal((K, N)) * 40), -128, 127).astype(np.int8)
        a_s = g.uniform(0.005, 0.02, rows).astype(np.float32)
        w_s = g.uniform(0.005, 0.02, N).astype(np.float32)
        total += timed(lambda: orc.gemm_w8a8(a, w, a_s, w_s)) * (M / rows)
        parts.append("C4 %d of 2048 rows" % rows)
    if which in ("all", "c5"):
        K, N, B, rows = 4096, 11008, 128, 4
        a = orc.narrow(g.standard_normal((rows, K), dtype=np.float32), orc.F16)
        wp = orc.pack_int4(g.integers(-8, 8, (K, N)).astype(np.int8))
        sc = orc.narrow(g.uniform(0.005, 0.02, (K // B, N)).astype(np.float32), orc.F16)
        orc.gemm_w4a16(a, wp, sc, K, N, B, mcount=0)                      # dequantised weights built once per call: time it apart
        t_deq = timed(lambda: orc.gemm_w4a16(a, wp, sc, K, N, B, mcount=0))
        t_rows = timed(lambda: orc.gemm_w4a16(a, wp, sc, K, N, B)) - t_deq
        total += 3 * t_deq + max(t_rows, 0.0) / rows * (16 + 256 + 4096)
        parts.append("C5 weight dequantisation in full + %d rows, scaled to M=16,256,4096" % rows)
    return total, ", ".join(parts)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="all", choices=["all", "c1", "c2a", "c2b", "c3", "c4", "c5", "nvfp4"])
    ap.add_argument("--settle-steps", type=int, default=100,
                    help="untimed steps in front of the warm-up, so that the timed steps run at the settled clocks (0: none)")
    ap.add_argument("--kernel-reps", type=int, default=100, help="launches per kernel for the per-kernel timing")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-cache-variants", action="store_true",
                    help="skip the warm-cache, 16x-rows and same-size yardstick launches (they reuse kernel names: keeps a profile's per-kernel averages clean)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every box of this build has one, and the hot path has no "
              "collective to time; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (there is no CPU fallback for the product path)", file=sys.stderr)
        sys.exit(2)
    pkg = entry.load_package()
    pkg.check(pkg.lib().mtrt_hip_init())
    torch.cuda.set_device(0)

    calibration_copy(pkg, torch)
    wl = build_workloads(pkg, torch, args.workload)
    # the step: every kernel once, in program order, on buffer set (step % nslots)
    step_calls = [[w["make"](i) for i in range(w["nslots"])] for w in wl]

    def run_step(k):
        for calls in step_calls:
            calls[k % len(calls)]()

    # Untimed lead-in before the warm-up: after an idle period (the set-up above leaves the GPU idle between its
    # launches) the board's power management needs some 10-15 ms of sustained load to settle: per-step times of a run
    # that starts cold read 695 666 675 698 751 778 755 701 709 678 671 668 665 665 ... us, so a window of 20 steps
    # right after 5 warm-up steps would time that transient, not the step.  The per-kernel figures below are taken in
    # steady state too (100 launches each, median of ten batches).
    for k in range(args.settle_steps):
        run_step(k)
    for k in range(args.warmup):
        run_step(k)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(args.steps):
        run_step(k)
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    ideal_us = 0.0
    kernels = []
    for w in wl:
        us = time_kernel(pkg, torch, w, args.kernel_reps)
        if w.get("dispatched"):              # the library chooses the kernel by shape: report the one it launched
            w["name"] = pkg.last_kernel()
        achieved = w["work"] / us / 1e3 if w["bound"] == "hbm" else w["work"] / us / 1e6
        ideal = w["work"] / (w["peak"] * 1e3) if w["bound"] == "hbm" else w["work"] / (w["peak"] * 1e6)
        ideal_us += ideal
        kernels.append(dict(kernel=w["name"], config=w["config"], bound=w["bound"], us=round(us, 2),
                            achieved=round(achieved, 1), peak=w["peak"], unit=w["unit"], frac=round(achieved / w["peak"], 4),
                            work=w["work"]))
    # what the matrix cores sustain on this very data with nothing else going on (power-limited)
    sustained, sustained_zero = {}, {}
    for w in wl:
        if w.get("probe"):
            kname, operand, ops = w["probe"]
            sustained[w["unit"]] = round(mfma_sustained(pkg, torch, kname, operand, ops), 1)
            # the yardstick's own ceiling: the same loop on all-zero operands (no toggling, full clock)
            sustained_zero[w["unit"]] = round(mfma_sustained(pkg, torch, kname, torch.zeros_like(operand), ops), 1)
    for k in kernels:
        if k["bound"] == "mfma" and k["unit"] in sustained:
            k["frac_of_sustained"] = round(k["achieved"] / sustained[k["unit"]], 4)
    # what the memory system sustains on this box (pure read, pure write, copy); HBM rows are also given as a fraction
    # of the yardstick with their access mix (amax only reads; every other cluster reads and writes, like the copy;
    # the small-M GEMM reads 60 bytes for every byte it writes)
    hbm, same_size = hbm_sustained(pkg, torch, [] if args.no_cache_variants else
                                   [(i, w["work"], w.get("mix", "copy")) for i, w in enumerate(wl) if w["bound"] == "hbm"], args.kernel_reps)
    for i, (w, k) in enumerate(zip(wl, kernels)):
        if k["bound"] == "hbm":
            mix = w.get("mix", "copy")
            k["frac_of_sustained"] = round(k["achieved"] / hbm[mix], 4)
            k["sustained_mix"] = mix
            if i in same_size:     # a plain read / copy launch moving the same number of bytes
                k["same_size_yardstick_us"] = same_size[i]
                k["frac_of_same_size_yardstick"] = round(same_size[i] / k["us"], 4)
    value = 100.0 * (ideal_us / 1e3) / ms_per_step
    dom = max(kernels, key=lambda k: k["us"])
    traffic = traffic_from_profile(dom["kernel"])
    line = {
        "metric": "Q/DQ+reduce HBM GB/s and W8A8/W4A16 GEMM TOPS, as % of MI355X peak, 1 GPU",
        "value": round(value, 2),
        "unit": "% of MI355X peak (time-weighted over the step's kernels)",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "settle_steps": args.settle_steps,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32 (Q/DQ, LayerNorm, softmax), int8->int32 (W8A8), f16->f32 (W4A16)", "data": "synthetic (seeded)",
        "config": {"workload": {"all": "C1+C2a+C2b+C3+C4+C5 programs of BASELINE.json, one pass each per step"}.get(
            args.workload, args.workload.upper()), "kernels_per_step": len(wl)},
        "roofline": {"kernel": dom["kernel"], "bound": dom["bound"], "achieved": dom["achieved"], "peak": dom["peak"],
                     "unit": dom["unit"], "frac": dom["frac"], "traffic": traffic[0], "traffic_source": traffic[1]},
        "mfma_sustained": {"rates": sustained, "rates_on_zero_operands": sustained_zero, "method": "mtrt_mfma_probe_*: 16 independent MFMAs per round and wave, one wave "
                           "per SIMD, operands = this bench's own data, no memory traffic; published dense peaks are "
                           "not reached on non-zero data (power limit)"},
        "hbm_sustained": {"rates": hbm, "unit": "GB/s", "method": "mtrt_read_b128 / mtrt_fill_b128 / mtrt_copy_b128 over 1 GiB per "
                          "stream: one 128-bit access per lane, one launch each, median of ten; copy counts bytes read + written"},
        "workloads": kernels,
    }
    if not args.no_cache_variants:
        for w, k in zip(wl, kernels):
            if w.get("zero_operands"):
                k["us_on_zero_operands"] = round(time_kernel(pkg, torch, dict(w, make=w["zero_operands"]), args.kernel_reps), 2)
    variants = [] if args.no_cache_variants else cache_variants(pkg, torch, wl, args.workload, args.kernel_reps)
    if variants:
        line["cache_variants"] = variants
    if not args.no_cache_variants and args.workload in ("all", "c4"):
        line["extra_clusters"] = extra_clusters(pkg, torch, args.kernel_reps)
    if not args.no_cache_variants:
        try:                      # an optional extra: never let the vendor library's state fail the benchmark
            yard = library_yardsticks(torch, args.workload, args.kernel_reps)
        except Exception as ex:   # noqa: BLE001
            yard = [dict(what="library yardsticks not available", error=str(ex)[:200])]
        if yard:
            line["library_yardsticks"] = yard
    if not args.no_cpu_baseline:
        cpu_s, sample = cpu_baseline(args.workload)
        line["cpu_baseline"] = {"value": round(100.0 * (ideal_us / 1e6) / cpu_s, 6),
                                "unit": "% of MI355X peak (same definition)", "cores": 1, "kind": "port",
                                "sample": sample + "; extrapolated linearly", "seconds_per_step": round(cpu_s, 3)}
        # the same sample with the oracle's OpenMP loops on every core this process may use (16 on the one-GPU box)
        cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
        cores = max(1, min(cores, int(os.environ.get("OMP_NUM_THREADS", cores))))
        cpu_all, _ = cpu_baseline(args.workload, cores)
        entry.load_oracle().set_threads(1)
        line["cpu_baseline_all_cores"] = {"value": round(100.0 * (ideal_us / 1e6) / cpu_all, 6),
                                          "unit": "% of MI355X peak (same definition)", "cores": cores, "kind": "port",
                                          "sample": "same sample, OpenMP over rows / tiles",
                                          "seconds_per_step": round(cpu_all, 3)}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
