// Host program written the way EmitC-generated C++ uses the StandaloneCPP runtime
// (mlir-tensorrt/compiler/test/IntegrationTests/EmitC/cuda-launch-argpack.mlir:84-130): it links
// against libmtrt_hip.so, calls the `namespace mtrt` functions declared in
// mtrt_hip_standalone.h and replays that test's known answer on the add_kernel fixture
// (args: in, out, u64 offset 4, u32 n 8, f32 2.5; expect out[4..11] = in + 2.5, the rest
// untouched).
//
//   standalone_selftest --validate           argument validation only, needs no device
//   standalone_selftest <fixtures.hsaco>     validation + the launch on the current device
#include <cstdio>
#include <cstring>
#include <string>

#include "mtrt_hip_standalone.h"

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
  EXPECT(cuda_module_create_from_ptx_file("/nonexistent/file.hsaco", &mod) == code(ErrorCode::IOError));
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
    std::fprintf(stderr, "usage: %s --validate | <fixtures.hsaco>\n", argv[0]);
    return 2;
  }
  if (validate() != 0)
    return 1;
  if (std::string(argv[1]) != "--validate" && launch_known_answer(argv[1]) != 0)
    return 1;
  std::printf("standalone selftest ok (%s)\n", argv[1]);
  return 0;
}
