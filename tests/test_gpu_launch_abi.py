"""Launch-ABI known answers, replayed through the C ABI with HIP rewrites of the
reference's two test kernels:
  mlir-tensorrt/compiler/test/IntegrationTests/CUDA/cuda-launch-kernel.mlir:60-110
  mlir-tensorrt/compiler/test/IntegrationTests/EmitC/cuda-launch-argpack.mlir:84-130
"""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _args(*cvals):
    arr = (ctypes.c_void_p * len(cvals))()
    for i, v in enumerate(cvals):
        arr[i] = ctypes.cast(ctypes.pointer(v), ctypes.c_void_p)
    return arr, cvals  # keep cvals alive


def _load_fixture_module(pkg, from_file):
    L = pkg.lib()
    if from_file:
        path = pkg.FIXTURE_MODULE_PATH.encode()
        return L.mtrt_cuda_module_load_from_ptx_file(path, len(path))
    data = open(pkg.FIXTURE_MODULE_PATH, "rb").read()
    return L.mtrt_cuda_module_load_from_ptx(data, len(data))


@pytest.mark.parametrize("from_file", [False, True])
def test_binary_shift_right_known_answer(pkg, from_file):
    import torch
    L = pkg.lib()
    mod = _load_fixture_module(pkg, from_file)
    assert mod
    name = b"binary_shift_rightXXXX"  # name is passed with an explicit length, not NUL-terminated
    fn = L.mtrt_cuda_module_get_function(mod, name, len(b"binary_shift_right"))
    assert fn
    stream = L.mtrt_cuda_stream_create()
    buf1 = torch.full((1, 32, 4), -1, dtype=torch.int32, device="cuda")
    buf2 = torch.zeros((1, 32, 4), dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    one_as_f32 = ctypes.c_float(np.array([1], dtype=np.int32).view(np.float32)[0])

    def launch(src, dst):
        args, keep = _args(ctypes.c_void_p(src.data_ptr()), ctypes.c_int32(7), one_as_f32,
                           ctypes.c_void_p(dst.data_ptr()))
        L.mtrt_cuda_launch_kernel(fn, 1, 1, 1, 32, 1, 1, 0, stream, args)
        L.mtrt_cuda_stream_sync(stream)

    launch(buf1, buf2)
    h = buf2.cpu().numpy()
    assert h[0, 0, 0] == 16777215 and h[0, 31, 3] == 16777215
    launch(buf2, buf1)
    h = buf1.cpu().numpy()
    assert h[0, 0, 0] == 65535 and h[0, 31, 3] == 65535
    L.mtrt_cuda_stream_destroy(stream)
    L.mtrt_cuda_module_unload(mod)


def test_argpack_known_answer(pkg):
    """(ptr, ptr, u64 offset=4, u32 n=8, f32 2.5): out[4..11] = in + 2.5, the rest untouched."""
    L = pkg.lib()
    mod = _load_fixture_module(pkg, True)
    fn = L.mtrt_cuda_module_get_function(mod, b"add_kernel", 10)
    stream = L.mtrt_cuda_stream_create()
    nbytes = 16 * 4
    in_dev = L.mtrt_cuda_alloc_async(stream, nbytes, 16, 0, 0)
    out_dev = L.mtrt_cuda_alloc_async(stream, nbytes, 16, 0, 0)
    in_host = L.mtrt_cuda_alloc_async(stream, nbytes, 16, 1, 0)
    out_host = L.mtrt_cuda_alloc_async(stream, nbytes, 16, 1, 0)
    hin = np.ctypeslib.as_array(ctypes.cast(in_host, ctypes.POINTER(ctypes.c_float)), shape=(16,))
    hout = np.ctypeslib.as_array(ctypes.cast(out_host, ctypes.POINTER(ctypes.c_float)), shape=(16,))
    hin[:] = np.arange(16, dtype=np.float32)
    hout[:] = np.arange(16, dtype=np.float32)
    L.mtrt_cuda_memcpy_async(stream, in_host, in_dev, nbytes)
    L.mtrt_cuda_memcpy_async(stream, out_host, out_dev, nbytes)
    args, keep = _args(ctypes.c_void_p(in_dev), ctypes.c_void_p(out_dev), ctypes.c_uint64(4),
                       ctypes.c_uint32(8), ctypes.c_float(2.5))
    L.mtrt_cuda_launch_kernel(fn, 1, 1, 1, 32, 1, 1, 0, stream, args)
    L.mtrt_cuda_memcpy_async(stream, out_dev, out_host, nbytes)
    L.mtrt_cuda_stream_sync(stream)
    expect = np.arange(16, dtype=np.float32)
    expect[4:12] += 2.5
    assert np.array_equal(hout, expect)
    L.mtrt_cuda_free(stream, in_dev, 0, 0)
    L.mtrt_cuda_free(stream, out_dev, 0, 0)
    L.mtrt_cuda_stream_sync(stream)
    L.mtrt_cuda_free(stream, in_host, 1, 0)
    L.mtrt_cuda_free(stream, out_host, 1, 0)
    L.mtrt_cuda_stream_destroy(stream)
    L.mtrt_cuda_module_unload(mod)


def test_events_and_devices(pkg):
    L = pkg.lib()
    dev = L.mtrt_cuda_get_current_device()
    assert dev == L.mtrt_cuda_get_active_device() == L.mtrt_cuda_get_program_device(0)
    assert L.mtrt_cuda_get_device(3) == 3
    assert L.mtrt_cuda_get_device_count() >= 1
    assert L.mtrt_cuda_set_active_device(dev) == dev
    s = L.mtrt_cuda_stream_create()
    e0, e1 = L.mtrt_cuda_event_create(dev), L.mtrt_cuda_event_create(dev)
    L.mtrt_cuda_stream_record_event(s, e0)
    L.mtrt_cuda_stream_record_event(s, e1)
    L.mtrt_cuda_stream_wait_event(s, e1)
    L.mtrt_cuda_event_sync(e1)
    assert L.mtrt_cuda_event_elapsed_msec(e0, e1) >= 0.0
    L.mtrt_cuda_event_release(e0)
    L.mtrt_cuda_event_release(e1)
    L.mtrt_cuda_stream_destroy(s)


def test_builtin_module_launch_through_part1(pkg, orc):
    """A cluster kernel launched by hand through module_load / get_function / launch_kernel with the argument
    array the reference's device ABI prescribes (ExpandMemRefArgs.cpp:65-120: bare pointers, i64 sizes, scalars by
    value): mtrt_q_uniform_f32_i8(x, q, scale, n, d1, nb, flags), seven operands of three widths, checked against
    the oracle; then the fused quantize+dequantize kernel the same way."""
    import numpy as np
    import torch
    L = pkg.lib()
    size = ctypes.c_size_t(0)
    blob = L.mtrt_hip_builtin_code_object(ctypes.byref(size))
    assert blob and size.value > 1000
    mod = L.mtrt_cuda_module_load_from_ptx(ctypes.string_at(blob, size.value), size.value)   # code object, not PTX
    assert mod
    rows, cols = 96, 4096
    x_np = np.random.Generator(np.random.PCG64(12)).standard_normal((rows, cols), dtype=np.float32)
    scale_np = np.float32(np.abs(x_np).max() / 127.0)
    x = torch.from_numpy(x_np).cuda()
    scale = torch.full((1,), float(scale_np), device="cuda")
    q = torch.zeros(rows * cols, dtype=torch.int8, device="cuda")
    n = rows * cols
    stream = torch.cuda.current_stream().cuda_stream
    name = b"mtrt_q_uniform_f32_i8"
    fn = L.mtrt_cuda_module_get_function(mod, name, len(name))
    args, keep = _args(ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(q.data_ptr()), ctypes.c_void_p(scale.data_ptr()),
                       ctypes.c_int64(n), ctypes.c_int64(cols), ctypes.c_int64(1), ctypes.c_int32(0))
    L.mtrt_cuda_launch_kernel(fn, (n + 4095) // 4096, 1, 1, 256, 1, 1, 0, stream, args)   # 256 lanes x 16 elements each
    torch.cuda.synchronize()
    q_ref = orc.quantize(x_np, orc.F32, orc.I8, [scale_np], orc.SCALE_UNIFORM, rows, cols)
    assert np.array_equal(q.cpu().numpy(), q_ref)
    # fused form: (x, q, y, scale, n, d1, nb, flags)
    y = torch.zeros_like(x)
    q.zero_()
    name = b"mtrt_qdq_uniform_f32_i8"
    fn2 = L.mtrt_cuda_module_get_function(mod, name, len(name))
    args2, keep2 = _args(ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(q.data_ptr()), ctypes.c_void_p(y.data_ptr()),
                         ctypes.c_void_p(scale.data_ptr()), ctypes.c_int64(n), ctypes.c_int64(cols), ctypes.c_int64(1),
                         ctypes.c_int32(0))
    L.mtrt_cuda_launch_kernel(fn2, (n + 4095) // 4096, 1, 1, 256, 1, 1, 0, stream, args2)
    torch.cuda.synchronize()
    assert np.array_equal(q.cpu().numpy(), q_ref)
    y_ref = orc.dequantize(q_ref, orc.I8, orc.F32, [scale_np], orc.SCALE_UNIFORM, rows, cols)
    assert np.array_equal(y.cpu().numpy().ravel().view(np.uint32), y_ref.view(np.uint32))
    L.mtrt_cuda_module_unload(mod)
