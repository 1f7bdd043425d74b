"""The two status-returning flavours of the launch layer.

  * `namespace mtrt` (include/mtrt_hip_standalone.h), the functions EmitC-generated host code calls in
    the reference (mlir-tensorrt/executor/lib/Runtime/StandaloneCPP/MTRTRuntimeCuda.h:36-110): exercised
    by a C++ host program linked against the library, built by build.py.
  * `mtrt_lua_cuda_*`, the bodies of the interpreter's `__cuda_*` builtins
    (mlir-tensorrt/executor/lib/Runtime/Backend/Lua/Modules/CUDA/CUDAModule.cpp:86-571): called through ctypes.

CPU tests cover exports and argument validation (no device call); GPU tests replay the reference's launch
known answers (mlir-tensorrt/compiler/test/IntegrationTests/EmitC/cuda-launch-argpack.mlir:84-130,
IntegrationTests/CUDA/cuda-launch-kernel.mlir:60-99)."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
STANDALONE_HEADER = os.path.join(ROOT, "include", "mtrt_hip_standalone.h")

# MTRTRuntimeCuda.h:36-110 and MTRTRuntimeStatus.h:48-53
REFERENCE_STANDALONE = [
    "cuda_get_current_device", "cuda_get_program_device", "cuda_stream_sync", "cuda_alloc", "cuda_free", "cuda_copy",
    "cuda_module_create_from_ptx_file", "cuda_module_destroy", "cuda_module_get_func", "cuda_launch_kernel",
    "cuda_event_create", "cuda_event_release", "cuda_stream_record_event", "cuda_stream_wait_event",
    "cuda_event_sync", "cuda_event_elapsed_msec", "get_last_error_message", "clear_last_error_message",
    # MTRTRuntimeStatus.h:55-58 and MTRTRuntimeCore.h:220-236 (abort_on_error, make_status and the memref
    # descriptor helpers are header-inline there and here: exercised by the selftest program)
    "set_last_error_message_v", "host_aligned_alloc", "host_free", "constant_load_from_file", "constant_destroy",
]


def _constant_env(tmp_path):
    """A 100-byte constant blob 0, 1, ..., 99 in a fresh artifacts directory, named through the environment."""
    (tmp_path / "weights.bin").write_bytes(bytes(range(100)))
    env = dict(os.environ)
    env["MTRT_ARTIFACTS_DIR"] = str(tmp_path)
    env["MTRT_SELFTEST_CONSTANT"] = "weights.bin"
    return env


def _selftest(pkg):
    return os.path.join(pkg.LIB_DIR, "mtrt_standalone_selftest")


def test_standalone_header_and_exports(pkg):
    text = re.sub(r"/\*.*?\*/", "", open(STANDALONE_HEADER).read(), flags=re.S)
    declared = re.findall(r"MTRT_CAPI_EXPORTED[^;(]*?\b([a-z_]+)\s*\(", text)
    assert sorted(declared) == sorted(REFERENCE_STANDALONE)
    out = subprocess.run(["nm", "-DC", "--defined-only", pkg.LIB_PATH], capture_output=True, text=True).stdout
    exported = set(re.findall(r" T mtrt::(?:detail::)?(\w+)\(", out))
    assert exported == set(REFERENCE_STANDALONE)
    # the header-inline part of the reference's interface
    for name in ("abort_on_error", "make_status", "make_memref_descriptor", "make_unranked_descriptor",
                 "make_ptr_shape_descriptor", "memref_descriptor_get_aligned_ptr", "memref_descriptor_get_stride",
                 "struct RankedMemRef", "struct UnrankedMemRef", "struct PtrAndShape", "bit_cast"):
        assert name in text, name
    # generated code includes the runtime under the reference's header names
    for shim in ("MTRTRuntimeStatus.h", "MTRTRuntimeCore.h", "MTRTRuntimeCuda.h"):
        assert os.path.exists(os.path.join(os.path.dirname(STANDALONE_HEADER), "standalone", shim))


def test_standalone_argument_validation(pkg, tmp_path):
    """null out-parameters, empty names, negative sizes, missing files, descriptor helpers, host-space constants
    from $MTRT_ARTIFACTS_DIR: status + message, no device needed."""
    res = subprocess.run([_selftest(pkg), "--validate"], capture_output=True, text=True, timeout=60,
                         env=_constant_env(tmp_path))
    assert res.returncode == 0, res.stdout + res.stderr
    assert "standalone selftest ok" in res.stdout


def test_abort_on_error_prints_the_message_and_aborts(pkg):
    """What generated code does after every runtime call (HostToEmitCPatternsCuda.cpp:39-42): a failed status
    prints the thread's last message to stderr and abort()s (MTRTRuntimeStatus.h:70-81)."""
    res = subprocess.run([_selftest(pkg), "--abort"], capture_output=True, text=True, timeout=60)
    assert res.returncode == -6, res.returncode
    assert "Error opening file 'mtrt_no_such_module.hsaco'" in res.stderr and "Tried:" in res.stderr


def test_builtin_name_table(pkg):
    L = pkg.lib()
    n = ctypes.c_size_t(0)
    table = L.mtrt_lua_cuda_builtins(ctypes.byref(n))
    entries = ctypes.cast(table, ctypes.POINTER(ctypes.c_char_p * 2 * n.value)).contents
    names = {bytes(e[0]).decode(): bytes(e[1]).decode() for e in entries}
    for lua_name in ("__cuda_load_module", "__cuda_get_function", "__cuda_launch", "__cuda_stream_create",
                     "__cuda_alloc_device", "__cuda_memcpy_host2device", "__cuda_memset_32",
                     "__cuda_get_program_device"):
        assert lua_name in names
    for sym in names.values():
        assert hasattr(L, sym), sym
    # every `__cuda_*` builtin the reference's CUDA module registers
    # (mlir-tensorrt/executor/lib/Runtime/Backend/Lua/Modules/CUDA/CUDAModule.cpp:86-571) has a body here
    reference_names = """__cuda_alloc_device __cuda_alloc_host_pinned __cuda_event_create __cuda_event_elapsed_msec
        __cuda_event_release __cuda_event_sync __cuda_free_device __cuda_free_host_pinned __cuda_get_active_device
        __cuda_get_device __cuda_get_function __cuda_get_program_device __cuda_launch __cuda_load_module
        __cuda_memcpy_device2device __cuda_memcpy_device2host __cuda_memcpy_device2host_pinned __cuda_memcpy_host2device
        __cuda_memcpy_host_pinned2device __cuda_memcpy_strided_async_device2device __cuda_memcpy_strided_async_device2host
        __cuda_memcpy_strided_async_device2host_pinned __cuda_memcpy_strided_async_host2device
        __cuda_memcpy_strided_async_host_pinned2device __cuda_memset_16 __cuda_memset_32 __cuda_memset_8 __cuda_num_devices
        __cuda_set_active_device __cuda_stream_create __cuda_stream_destroy __cuda_stream_record_event __cuda_stream_sync
        __cuda_stream_wait_event""".split()
    assert len(reference_names) == 34 and set(reference_names) == set(names)


def test_builtin_argument_validation(pkg):
    L = pkg.lib()
    out = ctypes.c_size_t(7)
    assert L.mtrt_lua_cuda_load_module(0, 0, 0, ctypes.byref(out)) == 1 and out.value == 0
    assert b"must not be empty" in L.mtrt_hip_last_error()
    assert L.mtrt_lua_cuda_load_module(0, 16, 16, None) == 1
    assert L.mtrt_lua_cuda_get_function(0, b"k", ctypes.byref(out)) == 1
    assert L.mtrt_lua_cuda_get_function(16, b"", ctypes.byref(out)) == 1
    assert L.mtrt_lua_cuda_launch(0, 1, 1, 1, 1, 1, 1, 0, 0, 16) == 1
    assert L.mtrt_lua_cuda_launch(16, 1, 1, 1, 1, 1, 1, 0, 0, 0) == 1
    assert L.mtrt_lua_cuda_memset(0, 16, 0, 16, 0, 3) == 1
    assert b"fill width" in L.mtrt_hip_last_error()
    assert L.mtrt_lua_cuda_memset(0, 16, 1, 16, 0, 4) == 1          # misaligned for a 32-bit pattern
    assert L.mtrt_lua_cuda_memset(0, 16, 0, 3, 0, 4) == 0           # fewer bytes than one element: nothing to do
    assert L.mtrt_lua_cuda_memcpy(0, 0, 0, 16, 0, 8) == 1
    assert L.mtrt_lua_cuda_memcpy(0, 0, 0, 0, 0, 0) == 0
    dev = ctypes.c_int32(-1)
    assert L.mtrt_lua_cuda_get_program_device(3, ctypes.byref(dev)) == 7
    assert b"out of range" in L.mtrt_hip_last_error()
    assert L.mtrt_lua_cuda_stream_destroy(0) == 1
    assert L.mtrt_lua_cuda_event_create(0, None) == 1
    assert L.mtrt_lua_cuda_event_release(0) == 0
    assert L.mtrt_lua_cuda_event_release(4096) == 1                  # not an event of the pool
    assert L.mtrt_lua_cuda_stream_record_event(0, 0) == 1
    ms = ctypes.c_float(1.0)
    assert L.mtrt_lua_cuda_event_elapsed_msec(0, 0, ctypes.byref(ms)) == 1
    p = ctypes.c_size_t(1)
    assert L.mtrt_lua_cuda_alloc_host_pinned(64, 3, ctypes.byref(p)) == 1 and p.value == 0
    assert L.mtrt_lua_cuda_alloc_host_pinned(64, 16, None) == 1
    assert L.mtrt_lua_cuda_free_host_pinned(0, 0) == 0
    shp = (ctypes.c_int64 * 4)(2, 3, 3, 1)
    bad = (ctypes.c_int64 * 4)(2, 4, 4, 1)
    assert L.mtrt_lua_cuda_memcpy_strided(0, 2, 4, 16, 0, shp, 16, 0, bad) == 1
    assert b"shapes differ" in L.mtrt_hip_last_error()
    assert L.mtrt_lua_cuda_memcpy_strided(0, 2, 0, 16, 0, shp, 16, 0, shp) == 1
    assert L.mtrt_lua_cuda_memcpy_strided(0, 2, 4, 0, 0, shp, 16, 0, shp) == 1


@pytest.mark.gpu
def test_standalone_launch_known_answer(pkg, tmp_path):
    """The reference's argpack known answer through the status-returning calls, then the same through functions
    written in the shape the EmitC lowering emits (alloc -> descriptor -> launch -> abort_on_error, copies of
    offset views), then constants loaded into the pinned, device and unified spaces."""
    print("case: standalone selftest on", pkg.FIXTURE_MODULE_PATH, flush=True)
    res = subprocess.run([_selftest(pkg), pkg.FIXTURE_MODULE_PATH], capture_output=True, text=True, timeout=100,
                         env=_constant_env(tmp_path))
    assert res.returncode == 0, res.stdout + res.stderr
    assert "standalone selftest ok" in res.stdout


@pytest.mark.gpu
def test_builtin_bodies_known_answers(pkg):
    """load_module from host bytes -> get_function -> launch with an argument-pointer array; memset, memcpy."""
    L = pkg.lib()
    sz = ctypes.c_size_t
    blob = open(pkg.FIXTURE_MODULE_PATH, "rb").read()
    buf = ctypes.create_string_buffer(blob, len(blob))
    mod, fn, stream = sz(0), sz(0), sz(0)
    dev = ctypes.c_int32(-1)
    assert L.mtrt_lua_cuda_get_program_device(0, ctypes.byref(dev)) == 0
    ndev = ctypes.c_int32(0)
    assert L.mtrt_lua_cuda_num_devices(ctypes.byref(ndev)) == 0 and ndev.value >= 1
    # PTX text is refused with a status, not an abort
    ptx = ctypes.create_string_buffer(b".version 7.0\n.target sm_80\n")
    assert L.mtrt_lua_cuda_load_module(dev.value, ctypes.addressof(ptx), len(ptx), ctypes.byref(mod)) == 1
    assert b"PTX is not accepted" in L.mtrt_hip_last_error()
    assert L.mtrt_lua_cuda_load_module(dev.value + 1, ctypes.addressof(buf), len(blob), ctypes.byref(mod)) == 1
    assert L.mtrt_lua_cuda_load_module(dev.value, ctypes.addressof(buf), len(blob), ctypes.byref(mod)) == 0, \
        L.mtrt_hip_last_error()
    assert L.mtrt_lua_cuda_get_function(mod.value, b"missing_kernel", ctypes.byref(fn)) == 4
    assert L.mtrt_lua_cuda_get_function(mod.value, b"binary_shift_right", ctypes.byref(fn)) == 0 and fn.value
    assert L.mtrt_lua_cuda_stream_create(ctypes.byref(stream)) == 0 and stream.value

    nbytes = 32 * 4 * 4
    a, b = sz(0), sz(0)
    assert L.mtrt_lua_cuda_alloc_device(stream.value, nbytes, ctypes.byref(a)) == 0 and a.value
    assert L.mtrt_lua_cuda_alloc_device(stream.value, nbytes, ctypes.byref(b)) == 0 and b.value
    # memset_32 with all ones, memset_8 zero (cuda-launch-kernel.mlir fills -1 and 0)
    assert L.mtrt_lua_cuda_memset(stream.value, a.value, 0, nbytes, 0xFFFFFFFF, 4) == 0
    assert L.mtrt_lua_cuda_memset(stream.value, b.value, 0, nbytes, 0, 1) == 0
    src, shift_i, dst = ctypes.c_void_p(a.value), ctypes.c_int32(7), ctypes.c_void_p(b.value)
    shift_f = ctypes.c_float(np.array([1], dtype=np.int32).view(np.float32)[0])
    slots = (src, shift_i, shift_f, dst)
    argv = (ctypes.c_void_p * 4)(*[ctypes.cast(ctypes.pointer(s), ctypes.c_void_p) for s in slots])
    assert L.mtrt_lua_cuda_launch(fn.value, 1, 1, 1, 32, 1, 1, 0, stream.value, ctypes.addressof(argv)) == 0
    host = np.zeros(32 * 4, dtype=np.int32)
    assert L.mtrt_lua_cuda_memcpy(stream.value, b.value, 0, host.ctypes.data, 0, nbytes) == 0
    assert L.mtrt_lua_cuda_stream_sync(stream.value) == 0
    assert np.all(host == 16777215)
    # 16-bit pattern on the second half only, through the offset argument
    assert L.mtrt_lua_cuda_memset(stream.value, b.value, nbytes // 2, nbytes // 2, 0xABCD, 2) == 0
    assert L.mtrt_lua_cuda_memcpy(stream.value, b.value, 0, host.ctypes.data, 0, nbytes) == 0
    assert L.mtrt_lua_cuda_stream_sync(stream.value) == 0
    assert np.all(host[:64] == 16777215) and np.all(host[64:].view(np.uint16) == 0xABCD)
    # a launch shape the device cannot run is a status
    assert L.mtrt_lua_cuda_launch(fn.value, 1, 1, 1, 4096, 1, 1, 0, stream.value, ctypes.addressof(argv)) == 4
    assert L.mtrt_lua_cuda_free_device(stream.value, a.value) == 0
    assert L.mtrt_lua_cuda_free_device(stream.value, b.value) == 0
    assert L.mtrt_lua_cuda_stream_sync(stream.value) == 0
    assert L.mtrt_lua_cuda_stream_destroy(stream.value) == 0


@pytest.mark.gpu
def test_builtin_events_pinned_memory_and_strided_copies(pkg):
    L = pkg.lib()
    sz = ctypes.c_size_t
    dev = L.mtrt_cuda_get_current_device()
    d = ctypes.c_int32(-1)
    assert L.mtrt_lua_cuda_get_active_device(ctypes.byref(d)) == 0 and d.value == dev
    assert L.mtrt_lua_cuda_set_active_device(dev) == 0
    assert L.mtrt_lua_cuda_get_device(0, ctypes.byref(d)) == 0 and d.value == dev
    assert L.mtrt_lua_cuda_set_active_device(4096) != 0 and L.mtrt_hip_last_error()
    stream, e0, e1, e2 = sz(0), sz(0), sz(0), sz(0)
    assert L.mtrt_lua_cuda_stream_create(ctypes.byref(stream)) == 0
    assert L.mtrt_lua_cuda_event_create(dev, ctypes.byref(e0)) == 0 and e0.value
    assert L.mtrt_lua_cuda_event_create(dev, ctypes.byref(e1)) == 0 and e1.value != e0.value
    # pinned staging buffers, 3 x 5 f32 matrix inside a 4 x 8 parent (row stride 8), copied to a dense device matrix
    hsrc, hdst, dbuf = sz(0), sz(0), sz(0)
    assert L.mtrt_lua_cuda_alloc_host_pinned(4 * 8 * 4, 64, ctypes.byref(hsrc)) == 0 and hsrc.value % 64 == 0
    assert L.mtrt_lua_cuda_alloc_host_pinned(6 * 5 * 4, 64, ctypes.byref(hdst)) == 0
    assert L.mtrt_lua_cuda_alloc_device(stream.value, 3 * 5 * 4, ctypes.byref(dbuf)) == 0
    src = np.ctypeslib.as_array(ctypes.cast(hsrc.value, ctypes.POINTER(ctypes.c_float)), shape=(4, 8))
    dst = np.ctypeslib.as_array(ctypes.cast(hdst.value, ctypes.POINTER(ctypes.c_float)), shape=(6, 5))
    src[:] = np.arange(32, dtype=np.float32).reshape(4, 8)
    dst[:] = -1.0
    strided = (ctypes.c_int64 * 4)(3, 5, 8, 1)
    dense = (ctypes.c_int64 * 4)(3, 5, 5, 1)
    every_other_row = (ctypes.c_int64 * 4)(3, 5, 10, 1)
    assert L.mtrt_lua_cuda_stream_record_event(stream.value, e0.value) == 0
    # host (offset: row 1, column 2) -> device, then device -> every other row of the host destination
    # offsets are memref offsets in ELEMENTS (reference: executor/lib/Support/StridedCopy.cpp:37-38)
    assert L.mtrt_lua_cuda_memcpy_strided(stream.value, 2, 4, hsrc.value, 1 * 8 + 2, strided, dbuf.value, 0, dense) == 0
    # ... and a non-zero destination offset of one row (5 elements): rows 1, 3, 5 of the destination
    assert L.mtrt_lua_cuda_memcpy_strided(stream.value, 2, 4, dbuf.value, 0, dense, hdst.value, 5, every_other_row) == 0
    # rank 0: exactly one element, element 3 of the device matrix -> element 2 of the host destination
    assert L.mtrt_lua_cuda_memcpy_strided(stream.value, 0, 4, dbuf.value, 3, None, hdst.value, 2, None) == 0
    assert L.mtrt_lua_cuda_stream_record_event(stream.value, e1.value) == 0
    assert L.mtrt_lua_cuda_stream_wait_event(stream.value, e1.value) == 0
    assert L.mtrt_lua_cuda_event_sync(e1.value) == 0
    ms = ctypes.c_float(-1.0)
    assert L.mtrt_lua_cuda_event_elapsed_msec(e0.value, e1.value, ctypes.byref(ms)) == 0 and ms.value >= 0.0
    expect = np.full((6, 5), -1.0, np.float32)
    expect[1::2] = src[1:4, 2:7]
    expect[0, 2] = src[1, 2 + 3]
    assert np.array_equal(dst, expect)
    # a released event comes back from the pool
    assert L.mtrt_lua_cuda_event_release(e1.value) == 0
    assert L.mtrt_lua_cuda_event_create(dev, ctypes.byref(e2)) == 0 and e2.value == e1.value
    assert L.mtrt_lua_cuda_event_release(e2.value) == 0 and L.mtrt_lua_cuda_event_release(e0.value) == 0
    # stream-ordered frees
    assert L.mtrt_lua_cuda_free_host_pinned(stream.value, hsrc.value) == 0
    assert L.mtrt_lua_cuda_free_host_pinned(stream.value, hdst.value) == 0
    assert L.mtrt_lua_cuda_free_device(stream.value, dbuf.value) == 0
    assert L.mtrt_lua_cuda_stream_sync(stream.value) == 0
    again = sz(0)
    assert L.mtrt_lua_cuda_alloc_host_pinned(128, 16, ctypes.byref(again)) == 0      # reaps the finished frees
    assert L.mtrt_lua_cuda_free_host_pinned(stream.value, again.value) == 0
    assert L.mtrt_lua_cuda_stream_sync(stream.value) == 0
    assert L.mtrt_lua_cuda_stream_destroy(stream.value) == 0


@pytest.mark.gpu
def test_strided_copies_between_device_addressable_views(pkg):
    """Views that the device can address on both sides are copied by one kernel (the reference issues a copy per
    element from the host, StridedCopy.cpp:57-75); results are those of indexing with the same shapes and strides."""
    import torch
    L = pkg.lib()
    stream = torch.cuda.current_stream().cuda_stream

    def copy(src, dst, shape, sstr, dstr, soff=0, doff=0, esize=None):
        rank = len(shape)
        s = (ctypes.c_int64 * (2 * rank))(*shape, *sstr)
        d = (ctypes.c_int64 * (2 * rank))(*shape, *dstr)
        pkg.check(L.mtrt_lua_cuda_memcpy_strided(stream, rank, esize or src.element_size(), src.data_ptr(), soff, s,
                                                 dst.data_ptr(), doff, d))

    g = torch.Generator(device="cuda").manual_seed(3)
    # transpose of a 300 x 500 f32 matrix: no two consecutive elements are contiguous on both sides
    a = torch.randn(300, 500, device="cuda", generator=g)
    t = torch.zeros(500, 300, device="cuda")
    copy(a, t, (500, 300), (1, 500), (300, 1))
    assert pkg.last_kernel() == "mtrt_copy_strided_b4"
    assert torch.equal(t, a.t())
    # rank 3, 2-byte elements, permuted source, destination a window (offset 7 elements) inside a larger buffer
    b = torch.randn(6, 10, 16, device="cuda", generator=g).to(torch.bfloat16)
    big = torch.zeros(4096, device="cuda", dtype=torch.bfloat16)
    copy(b, big, (10, 6, 16), (16, 160, 1), (6 * 20, 20, 1), doff=7)
    want = torch.zeros_like(big)
    want[7:7 + 10 * 120].view(10, 6, 20)[:, :, :16] = b.permute(1, 0, 2)
    assert torch.equal(big.view(torch.int16), want.view(torch.int16))
    # rows that are contiguous and 16-byte aligned move as 16-byte units; a negative row stride reverses the rows
    c = torch.arange(64 * 256, device="cuda", dtype=torch.float32).view(64, 256)
    r = torch.zeros(64, 128, device="cuda")
    copy(c, r, (64, 128), (-256, 1), (128, 1), soff=63 * 256 + 128)
    assert pkg.last_kernel() == "mtrt_copy_strided_b16"
    assert torch.equal(r, c.flip(0)[:, 128:])
    # 3-byte elements (units of one byte), pinned host source -> device destination with a gap between rows
    h = torch.arange(5 * 7 * 3, dtype=torch.uint8).pin_memory()
    d = torch.zeros(5 * 30, dtype=torch.uint8, device="cuda")
    copy(h, d, (5, 7), (7, 1), (10, 1), esize=3)
    assert pkg.last_kernel() == "mtrt_copy_strided_b1"
    torch.cuda.synchronize()
    want = torch.zeros(5, 30, dtype=torch.uint8)
    want[:, :21] = h.view(5, 21)
    assert torch.equal(d.cpu().view(5, 30), want)
    # ordinary (pageable) host memory on one side still goes run by run through the copy engine
    ph = np.arange(12, dtype=np.float32).reshape(3, 4)
    pd = torch.zeros(3, 2, device="cuda")
    s = (ctypes.c_int64 * 4)(3, 2, 4, 1)
    dd = (ctypes.c_int64 * 4)(3, 2, 2, 1)
    pkg.check(L.mtrt_lua_cuda_memcpy_strided(stream, 2, 4, ph.ctypes.data, 1, s, pd.data_ptr(), 0, dd))
    torch.cuda.synchronize()
    assert np.array_equal(pd.cpu().numpy(), ph[:, 1:3])
