// Host program written the way EmitC-generated C++ uses the StandaloneCPP runtime
// (mlir-tensorrt/compiler/test/IntegrationTests/EmitC/cuda-launch-argpack.mlir:84-130): it links
// against libmtrt_hip.so, calls the `namespace mtrt` functions declared in
// mtrt_hip_standalone.h and replays that test's known answer on the add_kernel fixture
// (args: in, out, u64 offset 4, u32 n 8, f32 2.5; expect out[4..11] = in + 2.5, the rest
// untouched).
//
//   standalone_selftest --validate           argument validation + host-side helpers, needs no device
//   standalone_selftest --abort              abort_on_error on a failed call: prints the message, aborts
//   standalone_selftest <fixtures.hsaco>     validation + the launches on the current device
//
// The generated-code shape is exercised literally: this file includes the runtime under the names generated
// code uses ("MTRTRuntimeCuda.h" etc., resolved through include/standalone) and spells handle types CUstream /
// CUfunction / CUmodule as the EmitC type converter does.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>

#include "MTRTRuntimeCore.h"
#include "MTRTRuntimeCuda.h"
#include "MTRTRuntimeStatus.h"

#define EXPECT(cond)                                                                                 \
  do {                                                                                               \
    if (!(cond)) {                                                                                   \
      std::fprintf(stderr, "FAILED %s:%d: %s | last error: %s\n", __FILE__, __LINE__, #cond,         \
                   mtrt::get_last_error_message());                                                  \
      return 1;                                                                                      \
    }                                                                                                \
  } while (false)

static int32_t code(mtrt::ErrorCode c) { return static_cast<int32_t>(c); }

static int validate() {
  using namespace mtrt;
  // null out-parameters and empty names: InvalidArgument with a message (MTRTRuntimeCuda.cpp:98-160)
  EXPECT(cuda_get_current_device(nullptr) == code(ErrorCode::InvalidArgument));
  EXPECT(std::strstr(get_last_error_message(), "outDevice must not be null"));
  clear_last_error_message();
  EXPECT(get_last_error_message()[0] == '\0');
  int32_t dev = -1;
  EXPECT(cuda_get_program_device(0, nullptr) == code(ErrorCode::InvalidArgument));
  EXPECT(cuda_get_program_device(1, &dev) == code(ErrorCode::InvalidArgument));
  EXPECT(std::strstr(get_last_error_message(), "logicalDevice must be 0"));
  EXPECT(cuda_get_program_device(0, &dev) == ok() && dev == 0);
  mtrt_module_t mod = reinterpret_cast<mtrt_module_t>(0x1);
  EXPECT(cuda_module_create_from_ptx_file("x", nullptr) == code(ErrorCode::InvalidArgument));
  EXPECT(cuda_module_create_from_ptx_file("", &mod) == code(ErrorCode::InvalidArgument) && mod == nullptr);
  // a missing artifact is NotFound and the message lists the places tried (MTRTRuntimeCore.cpp:76-93)
  EXPECT(cuda_module_create_from_ptx_file("/nonexistent/file.hsaco", &mod) == code(ErrorCode::NotFound));
  EXPECT(std::strstr(get_last_error_message(), "Tried:") && std::strstr(get_last_error_message(), "MTRT_ARTIFACTS_DIR"));
  mtrt_function_t fn = reinterpret_cast<mtrt_function_t>(0x1);
  EXPECT(cuda_module_get_func(nullptr, "k", nullptr) == code(ErrorCode::InvalidArgument));
  EXPECT(cuda_module_get_func(nullptr, "", &fn) == code(ErrorCode::InvalidArgument) && fn == nullptr);
  void *p = reinterpret_cast<void *>(0x1);
  EXPECT(cuda_alloc(nullptr, 16, false, false, nullptr) == code(ErrorCode::InvalidArgument));
  EXPECT(cuda_alloc(nullptr, -1, false, false, &p) == code(ErrorCode::InvalidArgument) && p == nullptr);
  EXPECT(cuda_alloc(nullptr, 0, false, false, &p) == ok() && p == nullptr);   // zero bytes: success, no pointer
  EXPECT(cuda_free(nullptr, nullptr, 0, 0) == ok());
  EXPECT(cuda_copy(nullptr, nullptr, nullptr, -4) == code(ErrorCode::InvalidArgument));
  EXPECT(cuda_copy(nullptr, nullptr, nullptr, 0) == ok());
  EXPECT(cuda_event_create(0, nullptr) == code(ErrorCode::InvalidArgument));
  EXPECT(cuda_event_release(nullptr) == ok());
  EXPECT(cuda_stream_record_event(nullptr, nullptr) == code(ErrorCode::InvalidArgument));
  EXPECT(cuda_stream_wait_event(nullptr, nullptr) == code(ErrorCode::InvalidArgument));
  EXPECT(cuda_event_sync(nullptr) == ok());
  float ms = 1.0f;
  EXPECT(cuda_event_elapsed_msec(nullptr, nullptr, nullptr) == code(ErrorCode::InvalidArgument));
  EXPECT(cuda_event_elapsed_msec(nullptr, nullptr, &ms) == code(ErrorCode::InvalidArgument) && ms == 0.0f);

  // status helpers and descriptors (MTRTRuntimeStatus.h:68-81, MTRTRuntimeCore.h:46-214)
  EXPECT(make_status(ErrorCode::NotFound) == 2 && make_status(ErrorCode::Success) == ok());
  abort_on_error(ok());                                     // returns
  detail::set_last_error_message("%s:%d", "where", 7);
  EXPECT(std::strcmp(get_last_error_message(), "where:7") == 0);
  EXPECT(bit_cast<uint32_t>(1.0f) == 0x3F800000u);
  int dummy[4] = {0, 0, 0, 0};
  auto m2 = make_memref_descriptor<2>(dummy, dummy + 1, 5, 3, 4, 8, 1);   // shape 3x4, strides 8,1, offset 5
  EXPECT(memref_descriptor_get_allocated_ptr(m2) == dummy && memref_descriptor_get_aligned_ptr(m2) == dummy + 1);
  EXPECT(memref_descriptor_get_offset(m2) == 5 && memref_descriptor_get_dim_size(m2, 0) == 3 &&
         memref_descriptor_get_dim_size(m2, 1) == 4 && memref_descriptor_get_stride(m2, 0) == 8 &&
         memref_descriptor_get_stride(m2, 1) == 1);
  auto m0 = make_memref_descriptor<0>(dummy, dummy, 0);
  EXPECT(memref_descriptor_get_offset(m0) == 0 && sizeof(m0) == 24 && sizeof(m2) == 24 + 2 * 2 * 8);
  UnrankedMemRef u = make_unranked_descriptor(2, m2);
  EXPECT(u.rank == 2 && u.rankedDescriptor == &m2);
  auto ps = make_ptr_shape_descriptor<2>(dummy, 3, 4);
  EXPECT(ps.bufferStart == dummy && memref_descriptor_get_dim_size(ps, 1) == 4);
  EXPECT(make_unranked_descriptor(2, ps).rankedDescriptor == &ps);
  EXPECT(make_unranked_descriptor_mut_ptr(2, &m2).rankedDescriptor == &m2);

  // host memory and host-space constants (MTRTRuntimeCore.cpp:246-358)
  void *h = reinterpret_cast<void *>(0x1);
  EXPECT(host_aligned_alloc(100, 0, &h) == code(ErrorCode::InvalidArgument) && h == nullptr);
  EXPECT(host_aligned_alloc(100, 48, &h) == code(ErrorCode::InvalidArgument));
  EXPECT(host_aligned_alloc(-1, 64, &h) == code(ErrorCode::InvalidArgument));
  EXPECT(host_aligned_alloc(0, 64, &h) == ok() && h == nullptr);
  EXPECT(host_aligned_alloc(100, 256, &h) == ok() && h && reinterpret_cast<uintptr_t>(h) % 256 == 0);
  host_free(h);
  EXPECT(constant_load_from_file("w.bin", 16, 1, nullptr) == code(ErrorCode::InvalidArgument));
  EXPECT(constant_load_from_file("", 16, 1, &h) == code(ErrorCode::InvalidArgument));
  EXPECT(constant_load_from_file("mtrt_no_such_constant.bin", 16, 1, &h) == code(ErrorCode::NotFound) && h == nullptr);
  if (const char *name = std::getenv("MTRT_SELFTEST_CONSTANT")) {
    // the caller wrote bytes 0, 1, 2, ... 99 into $MTRT_ARTIFACTS_DIR/<name>
    EXPECT(constant_load_from_file(name, 64, 1, &h) == ok() && h && reinterpret_cast<uintptr_t>(h) % 64 == 0);
    for (int i = 0; i < 100; ++i)
      EXPECT(static_cast<unsigned char *>(h)[i] == i);
    constant_destroy(h, 1);
    EXPECT(constant_load_from_file(name, 64, 9, &h) == code(ErrorCode::InvalidArgument));
  }
  constant_destroy(nullptr, 3);
  return 0;
}

// ---- functions in the shape the EmitC lowering emits ----------------------------------------------------
// cuda.alloc (HostToEmitCPatternsCuda.cpp:186-190): out pointer, call, abort_on_error, descriptor.
static mtrt::RankedMemRef<1> emitted_alloc(CUstream v1, int64_t v2) {
  int64_t v3 = 4;
  int64_t v4 = v2 * v3;
  void *v5 = nullptr;
  int32_t v6 = mtrt::cuda_alloc(v1, v4, false, false, &v5);
  mtrt::abort_on_error(v6);
  return mtrt::make_memref_descriptor<1>(v5, v5, 0, v2, 1);
}
// cuda.launch (HostToEmitCPatternsCuda.cpp:33-42): one local per operand, argv[] of their addresses.
static void emitted_launch(CUfunction v1, mtrt::RankedMemRef<1> v2, mtrt::RankedMemRef<1> v3, CUstream v4) {
  void *argv[5];
  void *v5 = mtrt::memref_descriptor_get_aligned_ptr(v2);
  argv[0] = (void *)&v5;
  void *v6 = mtrt::memref_descriptor_get_aligned_ptr(v3);
  argv[1] = (void *)&v6;
  int64_t v7 = 4;
  argv[2] = (void *)&v7;
  int32_t v8 = 8;
  argv[3] = (void *)&v8;
  float v9 = 2.5f;
  argv[4] = (void *)&v9;
  int32_t v10 = mtrt::cuda_launch_kernel(v1, 1, 1, 1, 32, 1, 1, 0, v4, argv);
  mtrt::abort_on_error(v10);
}
// cuda.copy_* of contiguous views with offsets (checked text: cuda-to-emitc.mlir, copy_d2h_offset).
static void emitted_copy(mtrt::RankedMemRef<1> v1, mtrt::RankedMemRef<1> v2, CUstream v3) {
  int64_t v4 = 4;
  int32_t v6 = 4;
  void *v7 = mtrt::memref_descriptor_get_aligned_ptr(v1);
  int8_t *v8 = (int8_t *)v7;
  int64_t v9 = mtrt::memref_descriptor_get_offset(v1);
  int64_t v10 = v9 * v6;
  void *v11 = v8 + v10;
  void *v12 = mtrt::memref_descriptor_get_aligned_ptr(v2);
  int8_t *v13 = (int8_t *)v12;
  int64_t v14 = mtrt::memref_descriptor_get_offset(v2);
  int64_t v15 = v14 * v6;
  void *v16 = v13 + v15;
  int64_t v17 = mtrt::memref_descriptor_get_dim_size(v1, 0) * v4;
  int32_t v18 = mtrt::cuda_copy(v3, v11, v16, v17);
  mtrt::abort_on_error(v18);
}
// cuda.dealloc
static void emitted_dealloc(CUstream v1, mtrt::RankedMemRef<1> v2) {
  int8_t v3 = 0;
  int8_t v4 = 0;
  void *v5 = mtrt::memref_descriptor_get_allocated_ptr(v2);
  int32_t v6 = mtrt::cuda_free(v1, v5, v3, v4);
  mtrt::abort_on_error(v6);
}

static int emitted_shape_known_answer(const char *fixture_path) {
  CUmodule mod = nullptr;
  mtrt::abort_on_error(mtrt::cuda_module_create_from_ptx_file(fixture_path, &mod));
  CUfunction fn = nullptr;
  mtrt::abort_on_error(mtrt::cuda_module_get_func(mod, "add_kernel", &fn));
  CUstream stream = mtrt_cuda_stream_create();
  mtrt::RankedMemRef<1> in = emitted_alloc(stream, 16), out = emitted_alloc(stream, 16);
  float host_in[16], host_out[16];
  for (int i = 0; i < 16; ++i) {
    host_in[i] = float(i);
    host_out[i] = -1.0f;
  }
  auto hin = mtrt::make_memref_descriptor<1>(host_in, host_in, 0, 16, 1);
  emitted_copy(hin, in, stream);
  emitted_copy(hin, out, stream);
  emitted_launch(fn, in, out, stream);
  // copy elements 4..11 of the result into elements 2..9 of the host buffer through offset views
  auto out_view = mtrt::make_memref_descriptor<1>(out.allocated, out.aligned, 4, 8, 1);
  auto host_view = mtrt::make_memref_descriptor<1>(host_out, host_out, 2, 8, 1);
  emitted_copy(out_view, host_view, stream);
  mtrt::abort_on_error(mtrt::cuda_stream_sync(stream));
  for (int i = 0; i < 16; ++i) {
    const float want = (i >= 2 && i < 10) ? float(i + 2) + 2.5f : -1.0f;
    if (host_out[i] != want) {
      std::fprintf(stderr, "FAILED (emitted shape): out[%d] = %g, expected %g\n", i, double(host_out[i]), double(want));
      return 1;
    }
  }
  emitted_dealloc(stream, in);
  emitted_dealloc(stream, out);
  mtrt::abort_on_error(mtrt::cuda_stream_sync(stream));

  // constants into the three device-visible spaces, read back through cuda_copy
  if (const char *name = std::getenv("MTRT_SELFTEST_CONSTANT")) {
    for (int32_t space : {2, 3, 4}) {
      void *c = nullptr;
      EXPECT(mtrt::constant_load_from_file(name, 16, space, &c) == mtrt::ok() && c);
      unsigned char back[100];
      std::memset(back, 0xEE, sizeof(back));
      EXPECT(mtrt::cuda_copy(stream, c, back, 100) == mtrt::ok());
      EXPECT(mtrt::cuda_stream_sync(stream) == mtrt::ok());
      for (int i = 0; i < 100; ++i)
        EXPECT(back[i] == i);
      mtrt::constant_destroy(c, space);
    }
  }
  mtrt::abort_on_error(mtrt::cuda_module_destroy(mod));
  mtrt_cuda_stream_destroy(stream);
  return 0;
}

static int launch_known_answer(const char *fixture_path) {
  using namespace mtrt;
  int32_t dev = -1;
  EXPECT(cuda_get_current_device(&dev) == ok() && dev >= 0);
  // a text file is not a code object
  mtrt_module_t mod = nullptr;
  EXPECT(cuda_module_create_from_ptx_file(__FILE__, &mod) != ok() && mod == nullptr);
  EXPECT(cuda_module_create_from_ptx_file(fixture_path, &mod) == ok() && mod);
  mtrt_function_t fn = nullptr;
  EXPECT(cuda_module_get_func(mod, "no_such_kernel", &fn) == code(ErrorCode::CUDADriverError) && fn == nullptr);
  EXPECT(cuda_module_get_func(mod, "add_kernel", &fn) == ok() && fn);

  mtrt_stream_t stream = mtrt_cuda_stream_create();
  const int64_t nbytes = 16 * sizeof(float);
  void *in_dev = nullptr, *out_dev = nullptr, *in_host = nullptr, *out_host = nullptr;
  EXPECT(cuda_alloc(stream, nbytes, false, false, &in_dev) == ok() && in_dev);
  EXPECT(cuda_alloc(stream, nbytes, false, false, &out_dev) == ok() && out_dev);
  EXPECT(cuda_alloc(stream, nbytes, true, false, &in_host) == ok() && in_host);
  EXPECT(cuda_alloc(stream, nbytes, false, true, &out_host) == ok() && out_host);
  float *hin = static_cast<float *>(in_host), *hout = static_cast<float *>(out_host);
  for (int i = 0; i < 16; ++i)
    hin[i] = hout[i] = float(i);
  EXPECT(cuda_copy(stream, in_host, in_dev, nbytes) == ok());
  EXPECT(cuda_copy(stream, out_host, out_dev, nbytes) == ok());

  mtrt_event_t e0 = nullptr, e1 = nullptr;
  EXPECT(cuda_event_create(dev, &e0) == ok() && e0);
  EXPECT(cuda_event_create(dev, &e1) == ok() && e1);
  EXPECT(cuda_stream_record_event(stream, e0) == ok());
  // one stack slot per operand, argv[] = their addresses (CUDAToExecutor.cpp:355-413)
  uint64_t offset = 4;
  uint32_t n = 8;
  float scalar = 2.5f;
  void *argv[] = {&in_dev, &out_dev, &offset, &n, &scalar};
  EXPECT(cuda_launch_kernel(fn, 1, 1, 1, 32, 1, 1, 0, stream, argv) == ok());
  EXPECT(cuda_stream_record_event(stream, e1) == ok());
  EXPECT(cuda_stream_wait_event(stream, e1) == ok());
  EXPECT(cuda_copy(stream, out_dev, out_host, nbytes) == ok());
  EXPECT(cuda_stream_sync(stream) == ok());
  EXPECT(cuda_event_sync(e1) == ok());
  float ms = -1.0f;
  EXPECT(cuda_event_elapsed_msec(e0, e1, &ms) == ok() && ms >= 0.0f);
  for (int i = 0; i < 16; ++i) {
    const float want = (i >= 4 && i < 12) ? float(i) + 2.5f : float(i);
    if (hout[i] != want) {
      std::fprintf(stderr, "FAILED: out[%d] = %g, expected %g\n", i, double(hout[i]), double(want));
      return 1;
    }
  }
  // an impossible launch shape is a status, not an abort
  EXPECT(cuda_launch_kernel(fn, 1, 1, 1, 4096, 1, 1, 0, stream, argv) == code(ErrorCode::CUDADriverError));
  EXPECT(get_last_error_message()[0] != '\0');

  EXPECT(cuda_event_release(e0) == ok() && cuda_event_release(e1) == ok());
  EXPECT(cuda_free(stream, in_dev, 0, 0) == ok() && cuda_free(stream, out_dev, 0, 0) == ok());
  EXPECT(cuda_stream_sync(stream) == ok());
  EXPECT(cuda_free(stream, in_host, 1, 0) == ok() && cuda_free(stream, out_host, 0, 1) == ok());
  EXPECT(cuda_module_destroy(mod) == ok());
  mtrt_cuda_stream_destroy(stream);
  return 0;
}

int main(int argc, char **argv) {
  if (argc != 2) {
    std::fprintf(stderr, "usage: %s --validate | --abort | <fixtures.hsaco>\n", argv[0]);
    return 2;
  }
  if (std::string(argv[1]) == "--abort") {
    // what generated code does after a failed call: message to stderr, then abort()
    CUmodule mod = nullptr;
    mtrt::abort_on_error(mtrt::cuda_module_create_from_ptx_file("mtrt_no_such_module.hsaco", &mod));
    return 0;   // not reached
  }
  if (validate() != 0)
    return 1;
  if (std::string(argv[1]) != "--validate" &&
      (launch_known_answer(argv[1]) != 0 || emitted_shape_known_answer(argv[1]) != 0))
    return 1;
  std::printf("standalone selftest ok (%s)\n", argv[1]);
  return 0;
}
