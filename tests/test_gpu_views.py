"""quantize / dequantize on strided rank-2 views (offset sub-tensors, row and column slices, transposes): results
equal the contiguous entry points on a packed copy and the oracle, bit for bit; one kernel is also launched by
hand with its operands in the order the reference expands dynamic memref arguments
(kernel/lib/Kernel/Transforms/ExpandMemRefArgs.cpp:65-120; compiler/test/Passes/1_Core/KernelToCUDA/kernel-to-cuda.mlir:3-48:
base, offset, size 0, size 1, stride 0, stride 1)."""
import ctypes

import numpy as np
import pytest

from helpers import bits16, rng

pytestmark = pytest.mark.gpu


def _views(parent):
    """name -> rank-2 view of the [40, 64] parent tensor"""
    return {
        "offset block": parent[3:27, 8:40],
        "every other row and column": parent[1::2, 0::2],
        "transpose": parent.t(),
        "single column": parent[:, 5:6],
        "whole": parent,
    }


@pytest.mark.parametrize("xname", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("qname", ["i8", "f8", "i4"])
def test_views_equal_packed_copies_and_the_oracle(pkg, orc, xname, qname):
    import torch
    td = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[xname]
    ox = {"f32": orc.F32, "bf16": orc.BF16, "f16": orc.F16}[xname]
    pq, oq = {"i8": (pkg.I8, orc.I8), "f8": (pkg.F8E4M3FN, orc.F8E4M3FN), "i4": (pkg.I4, orc.I4)}[qname]
    qmax = {"i8": 127.0, "f8": 448.0, "i4": 7.0}[qname]
    torch.manual_seed(3)
    parent = (torch.randn(40, 64, device="cuda") * 2).to(td)
    for name, xv in _views(parent).items():
        d0, d1 = xv.shape
        xc = xv.contiguous()
        xs = xc.cpu().numpy().ravel() if ox == orc.F32 else bits16(xc)
        for kind, okind, nb, ns in ((pkg.SCALE_UNIFORM, orc.SCALE_UNIFORM, 1, 1), (pkg.SCALE_ROW, orc.SCALE_ROW, d0, d0),
                                    (pkg.SCALE_COL, orc.SCALE_COL, d0, d1)):
            scale = (torch.rand(ns, device="cuda") * 0.05 + 0.01)
            # destination: a strided view as well (every second column of a wider buffer, after an offset)
            qbuf = torch.full((d0 + 2, 2 * d1 + 3), 0x55, dtype=torch.uint8, device="cuda")
            qv = qbuf[1:1 + d0, 3::2][:, :d1]
            pkg.quantize_view(xv, scale, pq, qv, kind, nb)
            # a source that runs fastest along its first dimension goes through 64 x 64 tiles, the rest one element per lane
            assert pkg.last_kernel() == "mtrt_q_view%s_%s_%s" % ("t" if name == "transpose" else "", xname, qname)
            q_ref = orc.quantize(xs, ox, oq, scale.cpu().numpy(), okind, d0, d1, nb)
            assert np.array_equal(qv.contiguous().cpu().numpy().ravel(), q_ref.view(np.uint8)), (name, kind)
            untouched = qbuf.clone()
            untouched[1:1 + d0, 3::2][:, :d1] = 0x55
            assert bool((untouched == 0x55).all()), "bytes outside the view were written (%s)" % name
            want = pkg.quantize(xc, scale, pq, kind, d0, d1, nb)
            assert torch.equal(qv.contiguous().view(torch.uint8).ravel(), want.view(torch.uint8).ravel())
            # dequantize the strided codes into a transposed destination
            ybuf = torch.zeros(d1, d0, dtype=td, device="cuda")
            pkg.dequantize_view(qv, scale, pq, ybuf.t(), kind, nb)
            assert pkg.last_kernel() == "mtrt_dq_viewt_%s_%s" % (xname, qname)
            y_ref = orc.dequantize(q_ref, oq, ox, scale.cpu().numpy(), okind, d0, d1, nb)
            got = ybuf.t().contiguous()
            got = got.cpu().numpy().ravel().view(np.uint32) if ox == orc.F32 else bits16(got)
            assert np.array_equal(got, y_ref.view(np.uint32) if ox == orc.F32 else y_ref), (name, kind)
            # ... and into every second column of a row-major buffer (no operand against the grain: one element per lane)
            ybuf2 = torch.full((d0, 2 * d1), 7.0, dtype=td, device="cuda")
            pkg.dequantize_view(qv, scale, pq, ybuf2[:, ::2], kind, nb)
            assert pkg.last_kernel() == "mtrt_dq_view_%s_%s" % (xname, qname)
            got2 = ybuf2[:, ::2].contiguous()
            got2 = got2.cpu().numpy().ravel().view(np.uint32) if ox == orc.F32 else bits16(got2)
            assert np.array_equal(got2, y_ref.view(np.uint32) if ox == orc.F32 else y_ref), (name, kind)
            assert bool((ybuf2[:, 1::2] == 7.0).all())


@pytest.mark.parametrize("xname", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("qname", ["i8", "f8", "i4"])
def test_views_with_contiguous_rows_take_the_row_walking_kernels(pkg, orc, xname, qname):
    """Row and column slices and offset sub-tensors keep their inner stride of one: both operands of such a call are
    walked row by row with vector accesses, the views' row strides as pitches.  Results against the oracle, nothing
    outside the destination views written; widths that are and are not whole vectors, a row step of two."""
    import torch
    td = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[xname]
    ox = {"f32": orc.F32, "bf16": orc.BF16, "f16": orc.F16}[xname]
    pq, oq = {"i8": (pkg.I8, orc.I8), "f8": (pkg.F8E4M3FN, orc.F8E4M3FN), "i4": (pkg.I4, orc.I4)}[qname]
    torch.manual_seed(11)
    parent = (torch.randn(70, 1200, device="cuda") * 2).to(td)
    views = {"offset block": parent[3:27, 8:40], "wide ragged slice": parent[1:60, 5:1136], "every other row": parent[1::2, 16:528],
             "whole": parent, "one column": parent[:, 7:8]}
    for name, xv in views.items():
        d0, d1 = xv.shape
        xc = xv.contiguous()
        xs = xc.cpu().numpy().ravel() if ox == orc.F32 else bits16(xc)
        for kind, okind, nb, ns, tag in ((pkg.SCALE_UNIFORM, orc.SCALE_UNIFORM, 1, 1, "rowu"), (pkg.SCALE_ROW, orc.SCALE_ROW, d0, d0, "rowu"),
                                         (pkg.SCALE_COL, orc.SCALE_COL, d0, d1, "colu")):
            scale = (torch.rand(ns, device="cuda") * 0.05 + 0.01)
            qbuf = torch.full((d0 + 2, d1 + 9), 0x55, dtype=torch.uint8, device="cuda")
            qv = qbuf[1:1 + d0, 5:5 + d1]
            pkg.quantize_view(xv, scale, pq, qv, kind, nb)
            assert pkg.last_kernel() == "mtrt_q_%s_%s_%s" % (tag, xname, qname), (name, pkg.last_kernel())
            q_ref = orc.quantize(xs, ox, oq, scale.cpu().numpy(), okind, d0, d1, nb)
            assert np.array_equal(qv.contiguous().cpu().numpy().ravel(), q_ref.view(np.uint8)), (name, kind)
            untouched = qbuf.clone()
            untouched[1:1 + d0, 5:5 + d1] = 0x55
            assert bool((untouched == 0x55).all()), "bytes outside the view were written (%s)" % name
            ybuf = torch.full((d0 + 1, d1 + 3), 7.0, dtype=td, device="cuda")
            yv = ybuf[1:, 2:2 + d1]
            pkg.dequantize_view(qv, scale, pq, yv, kind, nb)
            assert pkg.last_kernel() == "mtrt_dq_%s_%s_%s" % (tag, xname, qname)
            y_ref = orc.dequantize(q_ref, oq, ox, scale.cpu().numpy(), okind, d0, d1, nb)
            got = yv.contiguous()
            got = got.cpu().numpy().ravel().view(np.uint32) if ox == orc.F32 else bits16(got)
            assert np.array_equal(got, y_ref.view(np.uint32) if ox == orc.F32 else y_ref), (name, kind)
            rest = ybuf.clone()
            rest[1:, 2:2 + d1] = 7.0
            assert bool((rest == 7.0).all()), "values outside the destination view were written (%s)" % name


@pytest.mark.parametrize("xname", ["f32", "bf16"])
def test_dense_views_take_the_contiguous_kernels(pkg, orc, xname):
    """Views that are dense in both operands (whole row-major tensors with an offset, what a launch with memref
    descriptors usually passes) run the kernels of the contiguous entry points: the tile kernels when the offset
    pointers are aligned, the row-walking ones otherwise.  Same results as the oracle either way."""
    import torch
    td = {"f32": torch.float32, "bf16": torch.bfloat16}[xname]
    ox = {"f32": orc.F32, "bf16": orc.BF16}[xname]
    torch.manual_seed(12)
    d0, d1 = 96, 1024
    for off, tags in ((0, ("uniform", "row", "col")), (64, ("uniform", "row", "col")), (3, ("rowu", "rowu", "colu"))):
        xbuf = (torch.randn(off + d0 * d1, device="cuda") * 2).to(td)
        xv = xbuf[off:].view(d0, d1)
        xs = xv.cpu().numpy().ravel() if ox == orc.F32 else bits16(xv.contiguous())
        for (kind, okind, nb, ns), tag in zip(((pkg.SCALE_UNIFORM, orc.SCALE_UNIFORM, 1, 1), (pkg.SCALE_ROW, orc.SCALE_ROW, d0, d0),
                                              (pkg.SCALE_COL, orc.SCALE_COL, d0 // 32, 32 * d1)), tags):
            scale = torch.rand(ns, device="cuda") * 0.05 + 0.01
            qbuf = torch.full((off + d0 * d1 + 5,), 0x55, dtype=torch.uint8, device="cuda")
            qv = qbuf[off:off + d0 * d1].view(d0, d1)
            pkg.quantize_view(xv, scale, pkg.I8, qv, kind, nb)
            assert pkg.last_kernel() == "mtrt_q_%s_%s_i8" % (tag, xname), (off, kind, pkg.last_kernel())
            q_ref = orc.quantize(xs, ox, orc.I8, scale.cpu().numpy(), okind, d0, d1, nb)
            assert np.array_equal(qv.cpu().numpy().ravel(), q_ref.view(np.uint8))
            assert bool((qbuf[:off] == 0x55).all()) and bool((qbuf[off + d0 * d1:] == 0x55).all())
            ybuf = torch.full((off + d0 * d1 + 5,), 7.0, dtype=td, device="cuda")
            yv = ybuf[off:off + d0 * d1].view(d0, d1)
            pkg.dequantize_view(qv, scale, pkg.I8, yv, kind, nb)
            assert pkg.last_kernel() == "mtrt_dq_%s_%s_i8" % (tag, xname), (off, kind, pkg.last_kernel())
            y_ref = orc.dequantize(q_ref, orc.I8, ox, scale.cpu().numpy(), okind, d0, d1, nb)
            got = yv.cpu().numpy().ravel().view(np.uint32) if ox == orc.F32 else bits16(yv.contiguous())
            assert np.array_equal(got, y_ref.view(np.uint32) if ox == orc.F32 else y_ref)
            assert bool((ybuf[:off] == 7.0).all()) and bool((ybuf[off + d0 * d1:] == 7.0).all())


@pytest.mark.parametrize("xname", ["f32", "f16"])
@pytest.mark.parametrize("qname", ["i8", "f8"])
def test_transposed_views_go_through_tiles(pkg, orc, xname, qname):
    """Transposed sources into row-major codes, row-major codes into transposed destinations, both transposed, and a
    transposed slice with an offset: several 64 x 64 tiles with ragged edges, every scale kind, against the oracle;
    nothing outside the destination is written."""
    import torch
    td = {"f32": torch.float32, "f16": torch.float16}[xname]
    ox = {"f32": orc.F32, "f16": orc.F16}[xname]
    pq, oq = {"i8": (pkg.I8, orc.I8), "f8": (pkg.F8E4M3FN, orc.F8E4M3FN)}[qname]
    torch.manual_seed(21)
    parent = (torch.randn(200, 301, device="cuda") * 2).to(td)
    for name, xv in (("transpose", parent.t()), ("transposed slice", parent[5:133, 17:230].t()), ("row-major", parent)):
        d0, d1 = xv.shape
        xc = xv.contiguous()
        xs = xc.cpu().numpy().ravel() if ox == orc.F32 else bits16(xc)
        for kind, okind, nb, ns in ((pkg.SCALE_UNIFORM, orc.SCALE_UNIFORM, 1, 1), (pkg.SCALE_ROW, orc.SCALE_ROW, 7, 7),
                                    (pkg.SCALE_COL, orc.SCALE_COL, d0, d1)):
            scale = (torch.rand(ns, device="cuda") * 0.05 + 0.01)
            for q_transposed in (False, True):
                if name == "row-major" and not q_transposed:
                    continue                                     # dense on both sides: not a view kernel
                qbuf = torch.full((d1 + 2, d0 + 3) if q_transposed else (d0 + 2, d1 + 3), 0x55, dtype=torch.uint8, device="cuda")
                qv = qbuf[1:1 + d1, 2:2 + d0].t() if q_transposed else qbuf[1:1 + d0, 2:2 + d1]
                pkg.quantize_view(xv, scale, pq, qv, kind, nb)
                assert pkg.last_kernel() == "mtrt_q_viewt_%s_%s" % (xname, qname), (name, pkg.last_kernel())
                q_ref = orc.quantize(xs, ox, oq, scale.cpu().numpy(), okind, d0, d1, nb)
                assert np.array_equal(qv.contiguous().cpu().numpy().ravel(), q_ref.view(np.uint8)), (name, kind, q_transposed)
                rest = qbuf.clone()
                (rest[1:1 + d1, 2:2 + d0] if q_transposed else rest[1:1 + d0, 2:2 + d1])[:] = 0x55
                assert bool((rest == 0x55).all()), "bytes outside the view were written (%s)" % name
                ybuf = torch.full((d1 + 1, d0 + 2), 7.0, dtype=td, device="cuda")
                yv = ybuf[1:, 1:1 + d0].t()
                pkg.dequantize_view(qv, scale, pq, yv, kind, nb)
                assert pkg.last_kernel() == "mtrt_dq_viewt_%s_%s" % (xname, qname)
                y_ref = orc.dequantize(q_ref, oq, ox, scale.cpu().numpy(), okind, d0, d1, nb)
                got = yv.contiguous()
                got = got.cpu().numpy().ravel().view(np.uint32) if ox == orc.F32 else bits16(got)
                assert np.array_equal(got, y_ref.view(np.uint32) if ox == orc.F32 else y_ref), (name, kind, q_transposed)
                rest = ybuf.clone()
                rest[1:, 1:1 + d0] = 7.0
                assert bool((rest == 7.0).all())


def test_view_kernel_launched_by_hand_in_the_expanded_argument_order(pkg, orc):
    """memref<?x?xf32, strided<[?, ?], offset: ?>> -> (base, offset, size0, size1, stride0, stride1), per operand."""
    import torch
    L = pkg.lib()
    assert L.mtrt_hip_init() == 0
    parent = torch.from_numpy(rng(8).standard_normal((32, 48), dtype=np.float32)).cuda()
    xv = parent[4:20, 6:30:2]                                  # 16 x 12, offset 4*48+6, strides 48, 2
    q = torch.zeros(16, 12, dtype=torch.int8, device="cuda")
    scale = torch.full((1,), 0.03, device="cuda")
    name = b"mtrt_q_view_f32_i8"
    fn = L.mtrt_cuda_module_get_function(L.mtrt_hip_builtin_module(), name, len(name))
    i64, vp = ctypes.c_int64, ctypes.c_void_p
    vals = [vp(parent.data_ptr()), i64(4 * 48 + 6), i64(16), i64(12), i64(48), i64(2),
            vp(q.data_ptr()), i64(0), i64(16), i64(12), i64(12), i64(1),
            vp(scale.data_ptr()), i64(1), ctypes.c_int32(pkg.SCALE_UNIFORM), ctypes.c_int32(0)]
    args = (vp * len(vals))(*[ctypes.cast(ctypes.pointer(v), vp) for v in vals])
    L.mtrt_cuda_launch_kernel(fn, 1, 1, 1, 256, 1, 1, 0, torch.cuda.current_stream().cuda_stream, args)
    torch.cuda.synchronize()
    ref = orc.quantize(xv.contiguous().cpu().numpy().ravel(), orc.F32, orc.I8, [np.float32(scale.item())], orc.SCALE_UNIFORM, 16, 12)
    assert np.array_equal(q.cpu().numpy().ravel(), ref)


def test_view_argument_checks(pkg):
    import torch
    L = pkg.lib()
    x = torch.zeros(8, 8, device="cuda")
    q = torch.zeros(8, 8, dtype=torch.int8, device="cuda")
    s = torch.ones(1, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    ok = pkg.View2d(0, 8, 1)
    call = lambda xv, qv, qd=pkg.I8, kind=pkg.SCALE_UNIFORM, nb=1: L.mtrt_hip_quantize_view(
        st, x.data_ptr(), pkg.F32, ctypes.byref(xv), q.data_ptr(), qd, ctypes.byref(qv), s.data_ptr(), kind, 8, 8, nb, 0)
    assert call(ok, ok) == 0
    assert call(pkg.View2d(0, -8, 1), ok) == 1 and b"below its base" in L.mtrt_hip_last_error()
    assert call(pkg.View2d(56, -8, 1), ok) == 0                 # rows walked backwards from the last one: stays at or above the base
    assert call(ok, ok, pkg.I4_PACKED) == 1 and b"one code per byte" in L.mtrt_hip_last_error()
    assert call(ok, ok, pkg.I8, pkg.SCALE_COL, 3) == 1
    assert L.mtrt_hip_quantize_view(st, x.data_ptr(), pkg.F32, None, q.data_ptr(), pkg.I8, ctypes.byref(ok), s.data_ptr(), 0, 8, 8, 1, 0) == 1
