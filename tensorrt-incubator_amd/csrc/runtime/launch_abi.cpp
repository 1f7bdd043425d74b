// Part 1 of the C ABI: the executor runtime's kernel-launch layer on HIP.
// Same symbol names and argument lists as the reference C backend
// (mlir-tensorrt/executor/lib/Runtime/Backend/C/CUDAModule.cpp:57-252); the module
// entry points take a gfx950 code object where the reference takes PTX, so the
// nvPTXCompiler JIT step (mlir-tensorrt/executor/lib/Runtime/Backend/Common/
// NvPtxCompilerUtils.cpp:41-102) has no counterpart here.
#include "runtime_internal.hpp"

#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <string>
#include <vector>

namespace mtrt_rt {

[[noreturn]] void fatal(const char *file, int line, const char *msg) {
  std::fprintf(stderr, "%s#%d: %s\n", file, line, msg);
  std::fflush(stderr);
  std::abort();
}

bool read_file(const std::string &path, std::vector<char> &out) {
  std::ifstream in(path, std::ios::in | std::ios::binary);
  if (!in)
    return false;
  in.seekg(0, std::ios::end);
  const std::streamoff size = in.tellg();
  if (size < 0)
    return false;
  in.seekg(0, std::ios::beg);
  out.resize(static_cast<size_t>(size));
  if (size > 0)
    in.read(out.data(), size);
  return static_cast<bool>(in);
}

} // namespace mtrt_rt

using namespace mtrt_rt;

// Fatal-on-error, as HANDLE_CUDADRV_ERROR / HANDLE_CUDART_ERROR in the reference.
#define MTRT_FATAL_IF_HIP_ERROR(expr)                                                              \
  do {                                                                                             \
    hipError_t err_ = (expr);                                                                      \
    if (err_ != hipSuccess)                                                                        \
      fatal(__FILE__, __LINE__, hipGetErrorString(err_));                                          \
  } while (false)

extern "C" {

int32_t mtrt_cuda_get_active_device(void) {
  int device = 0;
  MTRT_FATAL_IF_HIP_ERROR(hipGetDevice(&device));
  return device;
}

int32_t mtrt_cuda_set_active_device(int32_t device) {
  MTRT_FATAL_IF_HIP_ERROR(hipSetDevice(device));
  return device;
}

int32_t mtrt_cuda_get_device(int32_t device) { return device; }

int32_t mtrt_cuda_get_device_count(void) {
  int count = 0;
  MTRT_FATAL_IF_HIP_ERROR(hipGetDeviceCount(&count));
  return count;
}

mtrt_stream_t mtrt_cuda_stream_create(void) {
  hipStream_t stream = nullptr;
  MTRT_FATAL_IF_HIP_ERROR(hipStreamCreate(&stream)); // default priority only
  return reinterpret_cast<mtrt_stream_t>(stream);
}

void mtrt_cuda_stream_destroy(mtrt_stream_t stream) {
  forget_stream(as_hip(stream));
  MTRT_FATAL_IF_HIP_ERROR(hipStreamDestroy(as_hip(stream)));
}

void mtrt_cuda_stream_sync(mtrt_stream_t stream) {
  MTRT_FATAL_IF_HIP_ERROR(hipStreamSynchronize(as_hip(stream)));
}

mtrt_event_t mtrt_cuda_event_create(int32_t device) {
  int current = -1;
  MTRT_FATAL_IF_HIP_ERROR(hipGetDevice(&current));
  if (current != device)
    MTRT_FATAL_IF_HIP_ERROR(hipSetDevice(device));
  hipEvent_t event = nullptr;
  MTRT_FATAL_IF_HIP_ERROR(hipEventCreateWithFlags(&event, hipEventDefault));
  if (current != device)
    MTRT_FATAL_IF_HIP_ERROR(hipSetDevice(current));
  return reinterpret_cast<mtrt_event_t>(event);
}

void mtrt_cuda_event_release(mtrt_event_t event) {
  MTRT_FATAL_IF_HIP_ERROR(hipEventDestroy(reinterpret_cast<hipEvent_t>(event)));
}

void mtrt_cuda_stream_record_event(mtrt_stream_t stream, mtrt_event_t event) {
  MTRT_FATAL_IF_HIP_ERROR(hipEventRecord(reinterpret_cast<hipEvent_t>(event), as_hip(stream)));
}

void mtrt_cuda_stream_wait_event(mtrt_stream_t stream, mtrt_event_t event) {
  MTRT_FATAL_IF_HIP_ERROR(
      hipStreamWaitEvent(as_hip(stream), reinterpret_cast<hipEvent_t>(event), /*flags=*/0));
}

void mtrt_cuda_event_sync(mtrt_event_t event) {
  MTRT_FATAL_IF_HIP_ERROR(hipEventSynchronize(reinterpret_cast<hipEvent_t>(event)));
}

float mtrt_cuda_event_elapsed_msec(mtrt_event_t start, mtrt_event_t end) {
  float ms = 0.0f;
  MTRT_FATAL_IF_HIP_ERROR(hipEventElapsedTime(&ms, reinterpret_cast<hipEvent_t>(start),
                                              reinterpret_cast<hipEvent_t>(end)));
  return ms;
}

void *mtrt_cuda_alloc_async(mtrt_stream_t stream, int64_t size, int32_t /*alignment*/,
                            int8_t isHostPinned, int8_t isManaged) {
  void *result = nullptr;
  if (isHostPinned || isManaged) {
    // Host-visible, device-visible memory.  Pinned host memory is allocated (not
    // registered) and serves both requests on a single-GPU node.
    MTRT_FATAL_IF_HIP_ERROR(hipHostMalloc(&result, static_cast<size_t>(size), hipHostMallocDefault));
    return result;
  }
  MTRT_FATAL_IF_HIP_ERROR(hipMallocAsync(&result, static_cast<size_t>(size), as_hip(stream)));
  return result;
}

void mtrt_cuda_memcpy_async(mtrt_stream_t stream, void *src, void *dest, int64_t size) {
  MTRT_FATAL_IF_HIP_ERROR(
      hipMemcpyAsync(dest, src, static_cast<size_t>(size), hipMemcpyDefault, as_hip(stream)));
}

void mtrt_cuda_free(mtrt_stream_t stream, void *ptr, int8_t isHostPinned, int8_t isManaged) {
  if (isHostPinned || isManaged) {
    MTRT_FATAL_IF_HIP_ERROR(hipHostFree(ptr));
    return;
  }
  MTRT_FATAL_IF_HIP_ERROR(hipFreeAsync(ptr, as_hip(stream)));
}

mtrt_module_t mtrt_cuda_module_load_from_ptx(const char *ptxData, size_t ptxLen) {
  hipModule_t module = nullptr;
  std::string err;
  if (load_code_object(ptxData, ptxLen, &module, &err) != MTRT_OK)
    fatal(__FILE__, __LINE__, err.c_str());
  return reinterpret_cast<mtrt_module_t>(module);
}

mtrt_module_t mtrt_cuda_module_load_from_ptx_file(const char *filename, size_t filenameLength) {
  const std::string path(filename, filenameLength);
  std::vector<char> bytes;
  if (!read_file(path, bytes)) {
    // The reference prints the failure and returns a null module here
    // (CUDAModule.cpp:201-203), leaving the crash to the first use.
    std::fprintf(stderr, "Error opening file '%s'.\n", path.c_str());
    return nullptr;
  }
  return mtrt_cuda_module_load_from_ptx(bytes.data(), bytes.size());
}

void mtrt_cuda_module_unload(mtrt_module_t module) {
  MTRT_FATAL_IF_HIP_ERROR(hipModuleUnload(reinterpret_cast<hipModule_t>(module)));
}

mtrt_function_t mtrt_cuda_module_get_function(mtrt_module_t module, const char *name,
                                              int64_t length) {
  hipFunction_t func = nullptr;
  const std::string name_(name, static_cast<size_t>(length));
  MTRT_FATAL_IF_HIP_ERROR(
      hipModuleGetFunction(&func, reinterpret_cast<hipModule_t>(module), name_.c_str()));
  return reinterpret_cast<mtrt_function_t>(func);
}

void mtrt_cuda_launch_kernel(mtrt_function_t func, int32_t gridX, int32_t gridY, int32_t gridZ,
                             int32_t blockX, int32_t blockY, int32_t blockZ,
                             int32_t dynamicSharedMemory, mtrt_stream_t stream, void **args) {
  // The reference writes "launching kernel:" to its debug stream on every call
  // (CUDAModule.cpp:231); that stream is off unless LLVM debugging is enabled, so
  // nothing is printed here.
  MTRT_FATAL_IF_HIP_ERROR(hipModuleLaunchKernel(
      reinterpret_cast<hipFunction_t>(func), uint32_t(gridX), uint32_t(gridY), uint32_t(gridZ),
      uint32_t(blockX), uint32_t(blockY), uint32_t(blockZ), uint32_t(dynamicSharedMemory),
      as_hip(stream), args, /*extra=*/nullptr));
}

int32_t mtrt_cuda_get_current_device(void) {
  int device = 0;
  MTRT_FATAL_IF_HIP_ERROR(hipGetDevice(&device));
  return device;
}

int32_t mtrt_cuda_get_program_device(int32_t logicalId) {
  if (logicalId != 0)
    fatal(__FILE__, __LINE__, "only single-device mode is supported");
  int device = 0;
  MTRT_FATAL_IF_HIP_ERROR(hipGetDevice(&device));
  return device;
}

} // extern "C"
