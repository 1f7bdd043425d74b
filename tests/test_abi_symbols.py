"""CPU-only checks of the drop-in boundary: the C-ABI library loads, exports exactly
the entry points include/mtrt_hip.h declares, keeps the reference C backend's names,
and carries a gfx950 code object with every kernel the cluster layer can ask for.
No compute call is made here."""
import ctypes
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mtrt_hip.h")

# names of the reference C backend, mlir-tensorrt/executor/lib/Runtime/Backend/C/CUDAModule.h:55-119
REFERENCE_C_BACKEND = [
    "mtrt_cuda_get_active_device", "mtrt_cuda_set_active_device", "mtrt_cuda_get_device",
    "mtrt_cuda_stream_create", "mtrt_cuda_stream_destroy", "mtrt_cuda_stream_sync",
    "mtrt_cuda_event_create", "mtrt_cuda_event_release", "mtrt_cuda_stream_record_event",
    "mtrt_cuda_stream_wait_event", "mtrt_cuda_event_sync", "mtrt_cuda_event_elapsed_msec",
    "mtrt_cuda_alloc_async", "mtrt_cuda_memcpy_async", "mtrt_cuda_free",
    "mtrt_cuda_module_load_from_ptx", "mtrt_cuda_module_load_from_ptx_file", "mtrt_cuda_module_unload",
    "mtrt_cuda_module_get_function", "mtrt_cuda_launch_kernel",
    "mtrt_cuda_get_current_device", "mtrt_cuda_get_program_device",
]


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"MTRT_CAPI_EXPORTED[^;(]*?\b(mtrt_[a-z0-9_]+)\s*\(", text)


def test_header_declares_the_reference_names():
    declared = _declared()
    assert len(declared) == len(set(declared))
    for name in REFERENCE_C_BACKEND:
        assert name in declared, name


def test_header_is_plain_c_and_carries_the_type_erased_twins(tmp_path):
    """Emitted C calls `<name>_cwrapper(void *...)` (reference CUDAModule.h:130-205): the header must compile
    as C and define one twin per wrapped entry point."""
    twins = ["stream_create", "stream_destroy", "stream_sync", "event_create", "event_release", "stream_record_event",
             "stream_wait_event", "event_sync", "event_elapsed_msec", "alloc_async", "memcpy_async", "free",
             "module_load_from_ptx", "module_load_from_ptx_file", "module_unload", "module_get_function",
             "launch_kernel", "get_current_device"]
    src = tmp_path / "twins.c"
    body = "".join("  p[%d] = (void *)&mtrt_cuda_%s_cwrapper;\n" % (i, t) for i, t in enumerate(twins))
    src.write_text('#include "mtrt_hip.h"\nvoid fill(void **p) {\n%s}\n' % body)
    out = subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Wno-pedantic", "-Werror", "-I", os.path.dirname(HEADER),
                          "-c", str(src), "-o", str(tmp_path / "twins.o")], capture_output=True, text=True)
    assert out.returncode == 0, out.stderr


def test_library_exports_every_declared_symbol(pkg):
    L = pkg.lib()
    for name in _declared():
        assert hasattr(L, name), "libmtrt_hip.so does not export %s" % name
    assert set(pkg.PROTOTYPES) == set(_declared()), "python prototypes and header disagree"
    out = subprocess.run(["nm", "-D", "--defined-only", pkg.LIB_PATH], capture_output=True, text=True).stdout
    exported = set(re.findall(r" T (\w+)", out))
    assert set(_declared()) <= exported
    extra = {s for s in exported if s.startswith("mtrt_")} - set(_declared())
    assert not extra, "exported but undeclared: %s" % sorted(extra)


def test_embedded_code_object_is_gfx950_and_has_the_kernels(pkg):
    L = pkg.lib()
    size = ctypes.c_size_t(0)
    ptr = L.mtrt_hip_builtin_code_object(ctypes.byref(size))
    blob = ctypes.string_at(ptr, size.value)
    assert blob == open(pkg.KERNEL_MODULE_PATH, "rb").read()
    assert blob.startswith(b"__CLANG_OFFLOAD_BUNDLE__") and b"gfx950" in blob[:4096]
    names = []
    for mode in ("q", "dq", "qdq"):
        for kind in ("uniform", "row", "col", "any"):
            for x in ("f32", "f16", "bf16"):
                for q in ("i8", "f8", "i4", "i4p", "f4p"):
                    names.append("mtrt_%s_%s_%s_%s" % (mode, kind, x, q))
    for mode in ("q", "dq", "qdq"):
        for kind in ("rowu", "colu"):
            for x in ("f32", "f16", "bf16"):
                for q in ("i8", "f8", "i4"):
                    names.append("mtrt_%s_%s_%s_%s" % (mode, kind, x, q))
    for x in ("f32", "f16", "bf16"):
        names.append("mtrt_amax_" + x)
        for v in ("v1", "v2", "v4", "v8", "v16", "any"):
            names += ["mtrt_layernorm_%s_%s" % (x, v), "mtrt_softmax_%s_%s" % (x, v)]
        names.append("mtrt_layernorm_%s_v8r" % x)
        # a workgroup per row (long rows), and the forms for rows that are not whole vectors / short rows
        for v in ("g256v8", "g256v16", "g1024v8", "g1024v16", "u8v1", "u16v1", "u32v1", "u64v1", "u64v2", "u64v4", "u64v8",
                  "u64v16", "u256v8", "u256v16", "u1024v8", "u1024v16"):
            names += ["mtrt_layernorm_%s_%s" % (x, v), "mtrt_softmax_%s_%s" % (x, v)]
        names += ["mtrt_amax_rows_" + x, "mtrt_amax_cols_" + x, "mtrt_amax_cols_split_" + x, "mtrt_amax_rows_split_" + x, "mtrt_amax_cols_u_" + x, "mtrt_amax_cols_split_u_" + x, "mtrt_amax_finish_" + x,
                  "mtrt_nvfp4_q_" + x, "mtrt_nvfp4_dq_" + x, "mtrt_nvfp4_qc_" + x, "mtrt_nvfp4_dqc_" + x]
        for q in ("i8", "f8", "i4"):
            names += ["mtrt_q_view_%s_%s" % (x, q), "mtrt_dq_view_%s_%s" % (x, q), "mtrt_q_viewt_%s_%s" % (x, q), "mtrt_dq_viewt_%s_%s" % (x, q)]
    names += ["mtrt_fill", "mtrt_gemm_dense_f32", "mtrt_gemm_dense_f16", "mtrt_gemm_dense_bf16", "mtrt_gemm_dense_mfma_f16", "mtrt_gemm_dense_mfma_bf16", "mtrt_gemm_dense_mfma_f32", "mtrt_gemm_dense_edge_f32", "mtrt_gemm_dense_edge_f16", "mtrt_gemm_dense_edge_bf16", "mtrt_gemm_w8a8_frag", "mtrt_gemm_w8a8_frag_t256x384",
              "mtrt_gemm_w8a8_small16", "mtrt_gemm_w8a8_frag_rows32", "mtrt_gemm_w8a8_nk", "mtrt_gemm_w8a8_nk_rows32", "mtrt_gemm_dense_rows32_f32", "mtrt_gemm_dense_rows32_f16", "mtrt_gemm_dense_rows32_bf16", "mtrt_gemm_w8a8_nk_rows64", "mtrt_gemm_w8a8_frag_rows64", "mtrt_gemm_w8a8_frag_rows128", "mtrt_gemm_w8a8_nk_rows128", "mtrt_gemm_dense_rows128_f32", "mtrt_gemm_dense_rows128_f16", "mtrt_gemm_dense_rows128_bf16", "mtrt_gemm_dense_rows64_f32", "mtrt_gemm_dense_rows64_f16", "mtrt_gemm_dense_rows64_bf16", "mtrt_gemm_w8a8_nk_edge", "mtrt_gemm_w8a8_nk_any", "mtrt_gemm_w4a16_t256x256", "mtrt_gemm_w4a16_t256x384",
              "mtrt_gemm_w4a16_t128x128", "mtrt_gemm_w4a16_t128x256", "mtrt_gemm_w4a16_t128x64", "mtrt_gemm_w4a16_skinny", "mtrt_gemm_w4a16_skinny16",
              "mtrt_gemm_w4a16_strips16", "mtrt_gemm_w4a16_edge", "mtrt_gemm_w4a16_any"]
    for n in names:
        assert n.encode() + b"\x00" in blob, "kernel %s is not in the code object" % n
    # measurement yardsticks and launch-ABI fixtures live in their own module, not in the product code object
    fixtures = open(pkg.FIXTURE_MODULE_PATH, "rb").read()
    for n in ("mtrt_copy_b128", "mtrt_mfma_probe_f16", "mtrt_mfma_probe_i8", "add_kernel", "binary_shift_right"):
        assert n.encode() + b"\x00" in fixtures and n.encode() + b"\x00" not in blob, n


def test_status_calls_fail_loudly_without_a_gpu(pkg):
    """There is no CPU fallback: without a usable gfx950 device init reports an error."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    L = pkg.lib()
    assert L.mtrt_hip_init() != 0
    assert L.mtrt_hip_last_error()
    assert L.mtrt_hip_builtin_module() is None
    st = L.mtrt_hip_softmax(None, 16, 16, pkg.F32, 1, 4)
    assert st != 0


def test_argument_validation_needs_no_device(pkg):
    L = pkg.lib()
    assert L.mtrt_hip_quantize(None, 16, 9, 16, pkg.I8, 16, 0, 1, 4, 1, 0) == 1
    assert b"f32/f16/bf16" in L.mtrt_hip_last_error()
    assert L.mtrt_hip_quantize(None, 16, pkg.F32, 16, pkg.I8, 16, 5, 1, 4, 1, 0) == 1
    assert L.mtrt_hip_quantize(None, 16, pkg.F32, 16, pkg.I8, 16, 0, -1, 4, 1, 0) == 1
    assert L.mtrt_hip_layernorm(None, 16, 16, 16, 16, pkg.I8, 1, 4, 1e-5) == 1
    assert L.mtrt_hip_amax(None, 16, pkg.F32, -5, 1.0, None, None) == 1
    # zero-sized work is a no-op that needs no device either
    assert L.mtrt_hip_quantize(None, 16, pkg.F32, 16, pkg.I8, 16, 0, 0, 4, 1, 0) == 0
    assert L.mtrt_hip_softmax(None, 16, 16, pkg.F32, 0, 4) == 0


def test_argument_validation_of_the_newer_entry_points_needs_no_device(pkg):
    """Every rejection below happens before the device is looked up, so it reads the same on a machine
    without a GPU; 16 stands for a non-null pointer that is never dereferenced."""
    import ctypes
    L = pkg.lib()
    err = lambda: L.mtrt_hip_last_error().decode()
    # amax per scale element
    assert L.mtrt_hip_amax_scales(None, 16, 9, pkg.SCALE_ROW, 4, 4, 4, 127.0, 16, 16) == 1 and "f32/f16/bf16" in err()
    assert L.mtrt_hip_amax_scales(None, 16, pkg.F32, 7, 4, 4, 4, 127.0, 16, 16) == 1 and "scale kind" in err()
    assert L.mtrt_hip_amax_scales(None, 16, pkg.F32, pkg.SCALE_ROW, 4, 4, 0, 127.0, 16, 16) == 1 and "positive" in err()
    assert L.mtrt_hip_amax_scales(None, 16, pkg.F32, pkg.SCALE_ROW, 4, 4, 5, 127.0, 16, 16) == 1 and "5 scales for 4 rows" in err()
    assert L.mtrt_hip_amax_scales(None, 16, pkg.F32, pkg.SCALE_COL, 6, 4, 4, 127.0, 16, 16) == 1 and "does not divide" in err()
    assert L.mtrt_hip_amax_scales(None, 16, pkg.F32, pkg.SCALE_COL, 8, 4, 4, 127.0, None, None) == 1 and "null operand" in err()
    assert L.mtrt_hip_amax_scales(None, 18, pkg.F32, pkg.SCALE_COL, 8, 4, 4, 127.0, 16, 16) == 1 and "aligned" in err()
    assert L.mtrt_hip_amax_scales(None, 16, pkg.F32, pkg.SCALE_COL, 0, 4, 4, 127.0, 16, 16) == 0      # nothing to reduce
    # dynamic quantization in one call
    dq = L.mtrt_hip_dynamic_quantize_dequantize
    assert dq(None, 16, pkg.F32, 16, pkg.I4, 16, 64, 127.0, 16, 16, 0) == 1 and "i8 or f8E4M3FN" in err()
    assert dq(None, 16, pkg.F32, 16, pkg.I8, 16, -1, 127.0, 16, 16, 0) == 1 and "negative" in err()
    assert dq(None, None, pkg.F32, 16, pkg.I8, 16, 64, 127.0, 16, 16, 0) == 1 and "null operand" in err()
    assert dq(None, 16, pkg.F32, 16, pkg.I8, 16, 64, 127.0, 16, None, 0) == 1 and "scale_out" in err()
    assert dq(None, 16, pkg.F32, 16, pkg.I8, 16, 64, 127.0, 16, 16, 64) == 1 and "flag" in err()
    # dynamic per-row quantization in one call
    dr = L.mtrt_hip_dynamic_quantize_rows
    assert dr(None, 16, 9, 16, pkg.I8, 4, 16, 127.0, 16, 16, 0) == 1 and "f32/f16/bf16" in err()
    assert dr(None, 16, pkg.F32, 16, pkg.I4, 4, 16, 7.0, 16, 16, 0) == 1 and "i8 or f8E4M3FN" in err()
    assert dr(None, 16, pkg.F32, 16, pkg.I8, -4, 16, 127.0, 16, 16, 0) == 1 and "negative" in err()
    assert dr(None, 16, pkg.F32, 16, pkg.I8, 1 << 20, 1 << 20, 127.0, 16, 16, 0) == 1 and "2^35" in err()
    assert dr(None, None, pkg.F32, 16, pkg.I8, 4, 16, 127.0, 16, 16, 0) == 1 and "null operand" in err()
    assert dr(None, 16, pkg.F32, 16, pkg.I8, 4, 16, 127.0, 16, None, 0) == 1 and "scale_out" in err()
    assert dr(None, 16, pkg.F32, 16, pkg.F8E4M3FN, 4, 16, 448.0, 16, 16, pkg.F8_REFHOST | pkg.F8_VIA_F16) == 1 and "two different" in err()
    assert dr(None, 16, pkg.F32, 16, pkg.I8, 0, 16, 127.0, 16, 16, 0) == 0                          # no rows
    # quantize on views
    ok_view = pkg.View2d(0, 8, 1)
    below = pkg.View2d(2, -8, 1)                               # row 1 would start 6 elements below the base pointer
    qv = L.mtrt_hip_quantize_view
    ref = ctypes.byref
    assert qv(None, 16, pkg.F32, ref(ok_view), 16, pkg.I4_PACKED, ref(ok_view), 16, pkg.SCALE_UNIFORM, 4, 8, 1, 0) == 1 and "one code per byte" in err()
    assert qv(None, 16, pkg.F32, None, 16, pkg.I8, ref(ok_view), 16, pkg.SCALE_UNIFORM, 4, 8, 1, 0) == 1 and "descriptor" in err()
    assert qv(None, 16, pkg.F32, ref(ok_view), 16, pkg.I8, ref(ok_view), 16, pkg.SCALE_COL, 6, 8, 4, 0) == 1 and "does not divide" in err()
    assert qv(None, 16, pkg.F32, ref(ok_view), 16, pkg.I8, ref(ok_view), 16, pkg.SCALE_UNIFORM, 4, 8, 1, pkg.F8_REFHOST | pkg.F8_VIA_F16) == 1 and "flag" in err()
    assert qv(None, 16, pkg.F32, ref(below), 16, pkg.I8, ref(ok_view), 16, pkg.SCALE_UNIFORM, 4, 8, 1, 0) == 1 and "below its base" in err()
    assert qv(None, 16, pkg.F32, ref(ok_view), 16, pkg.I8, ref(ok_view), 16, pkg.SCALE_UNIFORM, 1 << 20, 1 << 20, 1, 0) == 1 and "too large" in err()
    assert qv(None, 16, pkg.F32, ref(ok_view), 16, pkg.I8, ref(ok_view), 16, pkg.SCALE_UNIFORM, 0, 8, 1, 0) == 0
    # dense Linear
    ld = L.mtrt_hip_linear_dense
    assert ld(None, 16, 16, None, 16, 9, 4, 4, 4) == 1 and "f32/f16/bf16" in err()
    assert ld(None, 16, 16, None, 16, pkg.F16, 4, -4, 4) == 1 and "negative" in err()
    assert ld(None, 16, None, None, 16, pkg.F16, 4, 4, 4) == 1 and "null operand" in err()
    assert ld(None, 16, 16, 17, 16, pkg.F16, 4, 4, 4) == 1 and "aligned" in err()
    assert ld(None, 16, 16, None, 16, pkg.F16, 0, 4, 4) == 0
    # the block-wise GEMM and the size of its re-laid weights
    assert L.mtrt_hip_gemm_w4a16(None, 16, 16, 16, 16, 16, 4, 256, 64, 96) == 1 and "does not divide" in err()
    assert L.mtrt_hip_gemm_w4a16(None, 16, None, None, 16, 16, 4, 256, 64, 128) == 1 and "null operand" in err()
    assert L.mtrt_hip_gemm_w4a16_prepacked_bytes(4096, 11008) == 4096 * 11008            # two layouts of K*N/2 bytes each
    assert L.mtrt_hip_gemm_w4a16_prepacked_bytes(192, 64) == 192 * 64 // 2               # K % 128 != 0: fragment order only
    assert L.mtrt_hip_gemm_w4a16_prepacked_bytes(100, 64) == 0
    # the allocation-free reduction: its own limit, and it needs the library initialised on the device first
    assert L.mtrt_hip_amax_no_alloc(None, 16, pkg.F32, (1 << 36) + 1, 127.0, 16, 16) == 1 and "allocation-free amax accepts" in err()


def test_extents_whose_products_overflow_are_rejected(pkg):
    """Sizes are formed as products of 64-bit extents; extents that would overflow them are turned away first."""
    L = pkg.lib()
    big = 1 << 40
    assert L.mtrt_hip_quantize(None, 16, pkg.F32, 16, pkg.I8, 16, 0, big, big, 1, 0) == 1 and b"2^35" in L.mtrt_hip_last_error()
    assert L.mtrt_hip_amax_scales(None, 16, pkg.F32, pkg.SCALE_ROW, big, big, 4, 127.0, 16, 16) == 1
    assert L.mtrt_hip_softmax(None, 16, 16, pkg.F32, big, big) == 1
    assert L.mtrt_hip_layernorm(None, 16, 16, 16, 16, pkg.F32, big, big, 1e-5) == 1
    assert L.mtrt_hip_nvfp4_quantize(None, 16, pkg.F32, 16, 16, 16, big, big, 1) == 1
    assert L.mtrt_hip_gemm_w8a8(None, 16, 16, 16, 16, 16, 4, 1 << 31, 4) == 1 and b"2^31" in L.mtrt_hip_last_error()
    assert L.mtrt_hip_gemm_w4a16(None, 16, 16, 16, 16, 16, 1 << 31, 128, 4, 128) == 1
    assert L.mtrt_hip_linear_dense(None, 16, 16, None, 16, pkg.F16, 4, 4, 1 << 31) == 1
    assert L.mtrt_hip_gemm_w4a16_prepacked_bytes(1 << 32, 64) == 0
    assert L.mtrt_hip_gemm_w8a8_fragments_bytes(128, 1 << 31) == 0
