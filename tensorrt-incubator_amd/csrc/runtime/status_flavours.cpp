// The two status-returning flavours of the launch layer, over the same HIP calls as the fatal
// C entry points of launch_abi.cpp:
//
//  * `namespace mtrt` — what EmitC-generated host code calls in the reference's StandaloneCPP
//    runtime (mlir-tensorrt/executor/lib/Runtime/StandaloneCPP/MTRTRuntimeCuda.cpp:98-312):
//    null out-parameters and empty names are InvalidArgument, zero-size allocations and copies
//    succeed without touching the device, the message goes to a thread-local buffer.
//  * `mtrt_lua_cuda_*` — the bodies of the `__cuda_*` builtins the interpreter registers
//    (mlir-tensorrt/executor/lib/Runtime/Backend/Lua/Modules/CUDA/CUDAModule.cpp:86-571) with
//    handles as uintptr_t; a binding turns a non-zero status into a Lua error.
#include "mtrt_hip_standalone.h"
#include "runtime_internal.hpp"

#include <algorithm>
#include <cstring>
#include <map>
#include <mutex>
#include <utility>
#include <vector>

using namespace mtrt_rt;

namespace {

// The failure is reported through the status; the runtime's per-thread "last error" is cleared so
// that the caller's next, unrelated HIP call does not pick it up.
int32_t runtime_error(hipError_t e, const char *expr) {
  (void)hipGetLastError();
  return set_error(MTRT_RUNTIME_ERROR, "HIP runtime error: %s (%s)", hipGetErrorString(e), expr);
}
int32_t driver_error(hipError_t e, const char *expr) {
  (void)hipGetLastError();
  return set_error(MTRT_DRIVER_ERROR, "HIP module/launch error: %s (%s)", hipGetErrorString(e), expr);
}

#define RETURN_IF_RT(expr)                                                                         \
  do {                                                                                             \
    hipError_t e_ = (expr);                                                                        \
    if (e_ != hipSuccess)                                                                          \
      return runtime_error(e_, #expr);                                                             \
  } while (false)
#define RETURN_IF_DRV(expr)                                                                        \
  do {                                                                                             \
    hipError_t e_ = (expr);                                                                        \
    if (e_ != hipSuccess)                                                                          \
      return driver_error(e_, #expr);                                                              \
  } while (false)

hipEvent_t as_event(mtrt_event_t e) { return reinterpret_cast<hipEvent_t>(e); }

} // namespace

// ---------------------------------------------------------------------------
// namespace mtrt (StandaloneCPP flavour)
// ---------------------------------------------------------------------------
namespace mtrt {

const char *get_last_error_message() { return last_error(); }
void clear_last_error_message() { clear_error(); }

Status cuda_get_program_device(int32_t logicalDevice, int32_t *outDevice) {
  if (!outDevice)
    return set_error(MTRT_INVALID_ARGUMENT, "outDevice must not be null");
  if (logicalDevice != 0)
    return set_error(MTRT_INVALID_ARGUMENT, "logicalDevice must be 0, only SPMD mode is currently supported");
  *outDevice = 0;
  return ok();
}

Status cuda_module_create_from_ptx_file(const char *filename, mtrt_module_t *outModule) {
  if (!outModule)
    return set_error(MTRT_INVALID_ARGUMENT, "outModule must not be null");
  *outModule = nullptr;
  if (!filename || filename[0] == '\0')
    return set_error(MTRT_INVALID_ARGUMENT, "filename must not be empty");
  std::vector<char> bytes;
  const int32_t rd = read_artifact(filename, bytes);
  if (rd != MTRT_OK)
    return rd;
  hipModule_t module = nullptr;
  std::string err;
  const int32_t st = load_code_object(bytes.data(), bytes.size(), &module, &err);
  if (st != MTRT_OK)
    return set_error(st, "%s: %s", filename, err.c_str());
  *outModule = reinterpret_cast<mtrt_module_t>(module);
  return ok();
}

Status cuda_module_destroy(mtrt_module_t module) {
  RETURN_IF_DRV(hipModuleUnload(reinterpret_cast<hipModule_t>(module)));
  return ok();
}

Status cuda_module_get_func(mtrt_module_t module, const char *name, mtrt_function_t *outFunc) {
  if (!outFunc)
    return set_error(MTRT_INVALID_ARGUMENT, "outFunc must not be null");
  *outFunc = nullptr;
  if (!name || name[0] == '\0')
    return set_error(MTRT_INVALID_ARGUMENT, "name must not be empty");
  hipFunction_t f = nullptr;
  RETURN_IF_DRV(hipModuleGetFunction(&f, reinterpret_cast<hipModule_t>(module), name));
  *outFunc = reinterpret_cast<mtrt_function_t>(f);
  return ok();
}

Status cuda_launch_kernel(mtrt_function_t func, int32_t gridX, int32_t gridY, int32_t gridZ, int32_t blockX,
                          int32_t blockY, int32_t blockZ, int32_t dynamicSharedMemoryBytes,
                          mtrt_stream_t stream, void **arguments) {
  RETURN_IF_DRV(hipModuleLaunchKernel(reinterpret_cast<hipFunction_t>(func), uint32_t(gridX), uint32_t(gridY),
                                      uint32_t(gridZ), uint32_t(blockX), uint32_t(blockY), uint32_t(blockZ),
                                      uint32_t(dynamicSharedMemoryBytes), as_hip(stream), arguments, nullptr));
  return ok();
}

Status cuda_stream_sync(mtrt_stream_t stream) {
  RETURN_IF_RT(hipStreamSynchronize(as_hip(stream)));
  return ok();
}

Status cuda_get_current_device(int32_t *outDevice) {
  if (!outDevice)
    return set_error(MTRT_INVALID_ARGUMENT, "outDevice must not be null");
  int device = 0;
  RETURN_IF_RT(hipGetDevice(&device));
  *outDevice = device;
  return ok();
}

Status cuda_alloc(mtrt_stream_t stream, int64_t sizeBytes, bool isPinned, bool isManaged, void **outPtr) {
  if (!outPtr)
    return set_error(MTRT_INVALID_ARGUMENT, "outPtr must not be null");
  *outPtr = nullptr;
  if (sizeBytes < 0)
    return set_error(MTRT_INVALID_ARGUMENT, "sizeBytes must be >= 0");
  if (sizeBytes == 0)
    return ok();
  void *result = nullptr;
  if (isPinned || isManaged) {
    // Allocated (never registered) pinned host memory serves both requests on one GPU.
    RETURN_IF_RT(hipHostMalloc(&result, size_t(sizeBytes), hipHostMallocDefault));
  } else {
    RETURN_IF_RT(hipMallocAsync(&result, size_t(sizeBytes), as_hip(stream)));
  }
  *outPtr = result;
  return ok();
}

Status cuda_free(mtrt_stream_t stream, void *ptr, int8_t isHostPinned, int8_t isManaged) {
  if (!ptr)
    return ok();
  if (isHostPinned || isManaged) {
    RETURN_IF_RT(hipHostFree(ptr));
    return ok();
  }
  RETURN_IF_RT(hipFreeAsync(ptr, as_hip(stream)));
  return ok();
}

Status cuda_copy(mtrt_stream_t stream, void *src, void *dest, int64_t sizeBytes) {
  if (sizeBytes < 0)
    return set_error(MTRT_INVALID_ARGUMENT, "sizeBytes must be >= 0");
  if (sizeBytes == 0)
    return ok();
  RETURN_IF_RT(hipMemcpyAsync(dest, src, size_t(sizeBytes), hipMemcpyDefault, as_hip(stream)));
  return ok();
}

Status cuda_event_create(int32_t device, mtrt_event_t *outEvent) {
  if (!outEvent)
    return set_error(MTRT_INVALID_ARGUMENT, "outEvent must not be null");
  *outEvent = nullptr;
  int current = -1;
  RETURN_IF_RT(hipGetDevice(&current));
  if (current != device)
    RETURN_IF_RT(hipSetDevice(device));
  hipEvent_t event = nullptr;
  const hipError_t e = hipEventCreateWithFlags(&event, hipEventDefault);
  if (current != device)
    (void)hipSetDevice(current);
  if (e != hipSuccess)
    return runtime_error(e, "hipEventCreateWithFlags");
  *outEvent = reinterpret_cast<mtrt_event_t>(event);
  return ok();
}

Status cuda_event_release(mtrt_event_t event) {
  if (!event)
    return ok();
  RETURN_IF_RT(hipEventDestroy(as_event(event)));
  return ok();
}

Status cuda_stream_record_event(mtrt_stream_t stream, mtrt_event_t event) {
  if (!event)
    return set_error(MTRT_INVALID_ARGUMENT, "event must not be null");
  RETURN_IF_RT(hipEventRecord(as_event(event), as_hip(stream)));
  return ok();
}

Status cuda_stream_wait_event(mtrt_stream_t stream, mtrt_event_t event) {
  if (!event)
    return set_error(MTRT_INVALID_ARGUMENT, "event must not be null");
  RETURN_IF_RT(hipStreamWaitEvent(as_hip(stream), as_event(event), /*flags=*/0));
  return ok();
}

Status cuda_event_sync(mtrt_event_t event) {
  if (!event)
    return ok();
  RETURN_IF_RT(hipEventSynchronize(as_event(event)));
  return ok();
}

Status cuda_event_elapsed_msec(mtrt_event_t start, mtrt_event_t end, float *outMs) {
  if (!outMs)
    return set_error(MTRT_INVALID_ARGUMENT, "outMs must not be null");
  *outMs = 0.0f;
  if (!start || !end)
    return set_error(MTRT_INVALID_ARGUMENT, "start/end must not be null");
  RETURN_IF_RT(hipEventElapsedTime(outMs, as_event(start), as_event(end)));
  return ok();
}

} // namespace mtrt

// ---------------------------------------------------------------------------
// interpreter builtin bodies
// ---------------------------------------------------------------------------
extern "C" {

int32_t mtrt_lua_cuda_load_module(uint32_t device, uintptr_t data, uint64_t nbytes, uintptr_t *out_module) {
  if (!out_module)
    return set_error(MTRT_INVALID_ARGUMENT, "out_module must not be null");
  *out_module = 0;
  if (!data || nbytes == 0)
    return set_error(MTRT_INVALID_ARGUMENT, "module data must not be empty");
  int current = -1;
  RETURN_IF_RT(hipGetDevice(&current));
  if (uint32_t(current) != device)
    return set_error(MTRT_INVALID_ARGUMENT, "module requested for device %u while device %d is current", device,
                     current);
  hipModule_t module = nullptr;
  std::string err;
  const int32_t st = load_code_object(reinterpret_cast<const char *>(data), size_t(nbytes), &module, &err);
  if (st != MTRT_OK)
    return set_error(st, "%s", err.c_str());
  *out_module = reinterpret_cast<uintptr_t>(module);
  return MTRT_OK;
}

int32_t mtrt_lua_cuda_get_function(uintptr_t module, const char *name, uintptr_t *out_function) {
  mtrt_function_t f = nullptr;
  if (!out_function)
    return set_error(MTRT_INVALID_ARGUMENT, "out_function must not be null");
  *out_function = 0;
  if (!module)
    return set_error(MTRT_INVALID_ARGUMENT, "module must not be null");
  const int32_t st = mtrt::cuda_module_get_func(reinterpret_cast<mtrt_module_t>(module), name, &f);
  *out_function = reinterpret_cast<uintptr_t>(f);
  return st;
}

int32_t mtrt_lua_cuda_launch(uintptr_t func, int32_t gridX, int32_t gridY, int32_t gridZ, int32_t blockX,
                             int32_t blockY, int32_t blockZ, int32_t dynamicSharedMemory, uintptr_t stream,
                             uintptr_t argPtrArray) {
  if (!func)
    return set_error(MTRT_INVALID_ARGUMENT, "function must not be null");
  if (!argPtrArray)
    return set_error(MTRT_INVALID_ARGUMENT, "argument array must not be null");
  return mtrt::cuda_launch_kernel(reinterpret_cast<mtrt_function_t>(func), gridX, gridY, gridZ, blockX, blockY,
                                  blockZ, dynamicSharedMemory, reinterpret_cast<mtrt_stream_t>(stream),
                                  reinterpret_cast<void **>(argPtrArray));
}

int32_t mtrt_lua_cuda_stream_create(uintptr_t *out_stream) {
  if (!out_stream)
    return set_error(MTRT_INVALID_ARGUMENT, "out_stream must not be null");
  hipStream_t s = nullptr;
  *out_stream = 0;
  RETURN_IF_RT(hipStreamCreate(&s)); // default priority only
  *out_stream = reinterpret_cast<uintptr_t>(s);
  return MTRT_OK;
}

int32_t mtrt_lua_cuda_stream_sync(uintptr_t stream) {
  RETURN_IF_RT(hipStreamSynchronize(reinterpret_cast<hipStream_t>(stream)));
  return MTRT_OK;
}

int32_t mtrt_lua_cuda_stream_destroy(uintptr_t stream) {
  if (!stream)
    return set_error(MTRT_INVALID_ARGUMENT, "stream must not be null");
  forget_stream(reinterpret_cast<hipStream_t>(stream));
  RETURN_IF_RT(hipStreamDestroy(reinterpret_cast<hipStream_t>(stream)));
  return MTRT_OK;
}

int32_t mtrt_lua_cuda_alloc_device(uintptr_t stream, uint64_t nbytes, uintptr_t *out_ptr) {
  void *p = nullptr;
  if (!out_ptr)
    return set_error(MTRT_INVALID_ARGUMENT, "out_ptr must not be null");
  const int32_t st = mtrt::cuda_alloc(reinterpret_cast<mtrt_stream_t>(stream), int64_t(nbytes), false, false, &p);
  *out_ptr = reinterpret_cast<uintptr_t>(p);
  return st;
}

int32_t mtrt_lua_cuda_free_device(uintptr_t stream, uintptr_t ptr) {
  return mtrt::cuda_free(reinterpret_cast<mtrt_stream_t>(stream), reinterpret_cast<void *>(ptr), 0, 0);
}

int32_t mtrt_lua_cuda_memcpy(uintptr_t stream, uintptr_t src, uint64_t srcOffset, uintptr_t dst,
                             uint64_t dstOffset, uint64_t nbytes) {
  if (nbytes && (!src || !dst))
    return set_error(MTRT_INVALID_ARGUMENT, "src/dst must not be null");
  return mtrt::cuda_copy(reinterpret_cast<mtrt_stream_t>(stream), reinterpret_cast<void *>(src + srcOffset),
                         reinterpret_cast<void *>(dst + dstOffset), int64_t(nbytes));
}

int32_t mtrt_lua_cuda_memset(uintptr_t stream, uintptr_t ptr, uint64_t offset, uint64_t nbytes, uint32_t fill,
                             int32_t width) {
  if (width != 1 && width != 2 && width != 4)
    return set_error(MTRT_INVALID_ARGUMENT, "fill width must be 1, 2 or 4 bytes, got %d", width);
  uint8_t *p = reinterpret_cast<uint8_t *>(ptr + offset);
  if (nbytes && !ptr)
    return set_error(MTRT_INVALID_ARGUMENT, "pointer must not be null");
  if (reinterpret_cast<uintptr_t>(p) % uint32_t(width) != 0)
    return set_error(MTRT_INVALID_ARGUMENT, "pointer + offset is not aligned to the fill width %d", width);
  int64_t count = int64_t(nbytes / uint64_t(width)); // as the reference: numBytes / sizeof(fill)
  if (count == 0)
    return MTRT_OK;
  DeviceState *st = device_state();
  if (!st)
    return MTRT_RUNTIME_ERROR;
  const int64_t blocks = std::min<int64_t>((count + 255) / 256, int64_t(num_compute_units(st)) * 16);
  void *args[] = {&p, &count, &fill, &width};
  return launch(st, "mtrt_fill", uint32_t(blocks), 256, reinterpret_cast<hipStream_t>(stream), args);
}

// ---- events from a per-device pool -------------------------------------------------------------
namespace {
struct EventPool {
  std::mutex mu;
  std::map<int, std::vector<hipEvent_t>> free_by_device;
  std::map<hipEvent_t, int> device_of;                   // every event this pool ever created
};
EventPool &event_pool() {
  static EventPool *pool = new EventPool();              // never destroyed: events may outlive static teardown
  return *pool;
}
} // namespace

int32_t mtrt_lua_cuda_event_create(int32_t device, uintptr_t *out_event) {
  if (!out_event)
    return set_error(MTRT_INVALID_ARGUMENT, "out_event must not be null");
  *out_event = 0;
  EventPool &pool = event_pool();
  {
    std::lock_guard<std::mutex> lock(pool.mu);
    auto &free_list = pool.free_by_device[device];
    if (!free_list.empty()) {
      *out_event = reinterpret_cast<uintptr_t>(free_list.back());
      free_list.pop_back();
      return MTRT_OK;
    }
  }
  mtrt_event_t e = nullptr;
  const int32_t st = mtrt::cuda_event_create(device, &e);
  if (st != MTRT_OK)
    return st;
  std::lock_guard<std::mutex> lock(pool.mu);
  pool.device_of[reinterpret_cast<hipEvent_t>(e)] = device;
  *out_event = reinterpret_cast<uintptr_t>(e);
  return MTRT_OK;
}

int32_t mtrt_lua_cuda_event_release(uintptr_t event) {
  if (!event)
    return MTRT_OK;
  EventPool &pool = event_pool();
  std::lock_guard<std::mutex> lock(pool.mu);
  auto it = pool.device_of.find(reinterpret_cast<hipEvent_t>(event));
  if (it == pool.device_of.end())
    return set_error(MTRT_INVALID_ARGUMENT, "event was not created by mtrt_lua_cuda_event_create");
  pool.free_by_device[it->second].push_back(it->first);
  return MTRT_OK;
}

int32_t mtrt_lua_cuda_stream_record_event(uintptr_t stream, uintptr_t event) {
  return mtrt::cuda_stream_record_event(reinterpret_cast<mtrt_stream_t>(stream), reinterpret_cast<mtrt_event_t>(event));
}
int32_t mtrt_lua_cuda_stream_wait_event(uintptr_t stream, uintptr_t event) {
  return mtrt::cuda_stream_wait_event(reinterpret_cast<mtrt_stream_t>(stream), reinterpret_cast<mtrt_event_t>(event));
}
int32_t mtrt_lua_cuda_event_sync(uintptr_t event) { return mtrt::cuda_event_sync(reinterpret_cast<mtrt_event_t>(event)); }
int32_t mtrt_lua_cuda_event_elapsed_msec(uintptr_t start, uintptr_t end, float *out_ms) {
  return mtrt::cuda_event_elapsed_msec(reinterpret_cast<mtrt_event_t>(start), reinterpret_cast<mtrt_event_t>(end), out_ms);
}

// ---- pinned host memory with stream-ordered release -------------------------------------------
namespace {
struct PinnedFrees {
  std::mutex mu;
  std::vector<std::pair<hipEvent_t, void *>> pending;    // block is free once the event has completed
};
PinnedFrees &pinned_frees() {
  static PinnedFrees *p = new PinnedFrees();
  return *p;
}
// releases every block whose stream has passed the point of its free call
void reap_pinned(bool wait) {
  PinnedFrees &pf = pinned_frees();
  std::lock_guard<std::mutex> lock(pf.mu);
  size_t keep = 0;
  for (auto &entry : pf.pending) {
    const hipError_t q = wait ? hipEventSynchronize(entry.first) : hipEventQuery(entry.first);
    if (q == hipSuccess) {
      (void)hipEventDestroy(entry.first);
      (void)hipHostFree(entry.second);
    } else {
      if (q != hipErrorNotReady)
        (void)hipGetLastError();
      pf.pending[keep++] = entry;
    }
  }
  pf.pending.resize(keep);
}
} // namespace

int32_t mtrt_lua_cuda_alloc_host_pinned(uint64_t nbytes, int32_t alignment, uintptr_t *out_ptr) {
  if (!out_ptr)
    return set_error(MTRT_INVALID_ARGUMENT, "out_ptr must not be null");
  *out_ptr = 0;
  if (alignment <= 0 || (alignment & (alignment - 1)) != 0)
    return set_error(MTRT_INVALID_ARGUMENT, "alignment must be a positive power of two, got %d", alignment);
  reap_pinned(false);
  if (nbytes == 0)
    return MTRT_OK;
  void *p = nullptr;
  RETURN_IF_RT(hipHostMalloc(&p, size_t(nbytes), hipHostMallocDefault));
  if (reinterpret_cast<uintptr_t>(p) % uint32_t(alignment) != 0) {
    (void)hipHostFree(p);
    return set_error(MTRT_INTERNAL_ERROR, "allocated host pinned pointer %p does not have desired alignment %d", p, alignment);
  }
  *out_ptr = reinterpret_cast<uintptr_t>(p);
  return MTRT_OK;
}

int32_t mtrt_lua_cuda_free_host_pinned(uintptr_t stream, uintptr_t ptr) {
  if (!ptr)
    return MTRT_OK;
  hipEvent_t e = nullptr;
  RETURN_IF_RT(hipEventCreateWithFlags(&e, hipEventDisableTiming));
  const hipError_t r = hipEventRecord(e, reinterpret_cast<hipStream_t>(stream));
  if (r != hipSuccess) {
    (void)hipEventDestroy(e);
    return runtime_error(r, "hipEventRecord");
  }
  {
    PinnedFrees &pf = pinned_frees();
    std::lock_guard<std::mutex> lock(pf.mu);
    pf.pending.emplace_back(e, reinterpret_cast<void *>(ptr));
  }
  reap_pinned(false);
  return MTRT_OK;
}

// ---- strided copies --------------------------------------------------------------------------
int32_t mtrt_lua_cuda_memcpy_strided(uintptr_t stream, int64_t rank, int64_t elemSize, uintptr_t src, uint64_t srcOffset,
                                     const int64_t *srcShapeAndStrides, uintptr_t dst, uint64_t dstOffset,
                                     const int64_t *dstShapeAndStrides) {
  if (rank < 0 || rank > 16 || elemSize <= 0)
    return set_error(MTRT_INVALID_ARGUMENT, "rank %lld / element size %lld out of range", (long long)rank, (long long)elemSize);
  if (rank > 0 && (!srcShapeAndStrides || !dstShapeAndStrides))
    return set_error(MTRT_INVALID_ARGUMENT, "shape/stride arrays must not be null");
  if (!src || !dst)
    return set_error(MTRT_INVALID_ARGUMENT, "src/dst must not be null");
  const int64_t *shape = srcShapeAndStrides, *ss = srcShapeAndStrides + rank, *ds = dstShapeAndStrides + rank;
  int64_t total = 1;
  bool empty = false;
  for (int64_t i = 0; i < rank; ++i) {
    if (shape[i] != dstShapeAndStrides[i])
      return set_error(MTRT_INVALID_ARGUMENT, "source and destination shapes differ in dimension %lld", (long long)i);
    if (shape[i] < 0)
      return set_error(MTRT_INVALID_ARGUMENT, "negative extent in dimension %lld", (long long)i);
    empty = empty || shape[i] == 0;
    if (!empty && (__builtin_mul_overflow(total, shape[i], &total) || total >= (int64_t(1) << 48)))
      return set_error(MTRT_INVALID_ARGUMENT, "shape is too large for one copy");
  }
  if (empty)
    return MTRT_OK;
  if (elemSize > (int64_t(1) << 14))
    return set_error(MTRT_INVALID_ARGUMENT, "element size %lld out of range", (long long)elemSize);
  // innermost dimensions that are densely packed in BOTH operands form one contiguous run
  int64_t run = 1, inner = rank;
  while (inner > 0 && ss[inner - 1] == run && ds[inner - 1] == run) {
    run *= shape[inner - 1];
    --inner;
  }
  // offsets are memref offsets, in ELEMENTS (mlir-tensorrt/executor/lib/Support/StridedCopy.cpp:37-38)
  const char *sbase = reinterpret_cast<const char *>(src) + int64_t(srcOffset) * elemSize;
  char *dbase = reinterpret_cast<char *>(dst) + int64_t(dstOffset) * elemSize;
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
  if (inner == 0) {                                    // dense on both sides: one copy
    RETURN_IF_RT(hipMemcpyAsync(dbase, sbase, size_t(run * elemSize), hipMemcpyDefault, hs));
    return MTRT_OK;
  }

  // Both views in memory the device can address (device memory, pinned or managed host memory): one kernel walks
  // the index space.  The unit it moves is the largest power of two up to 16 bytes that divides the run, every
  // outer stride and both base addresses; the units of a run become the innermost dimension.
  auto device_can_address = [](const void *p) {
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
      (void)hipGetLastError();                           // ordinary host memory: not an error of this call
      return false;
    }
    return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeHost || attr.type == hipMemoryTypeManaged ||
           attr.type == hipMemoryTypeUnified;
  };
  if (inner <= 7 && device_can_address(sbase) && device_can_address(dbase)) {
    const int64_t run_bytes = run * elemSize;
    uint64_t bits = uint64_t(run_bytes) | reinterpret_cast<uintptr_t>(sbase) | reinterpret_cast<uintptr_t>(dbase) | 16u;
    for (int64_t i = 0; i < inner; ++i)
      if (shape[i] > 1)
        bits |= uint64_t(ss[i] * elemSize) | uint64_t(ds[i] * elemSize);
    const int64_t unit = int64_t(bits & (~bits + 1));     // lowest set bit: 1, 2, 4, 8 or 16
    struct {
      int64_t extent[8], src_stride[8], dst_stride[8];
    } sh = {};
    int32_t krank = int32_t(inner) + 1;
    for (int64_t i = 0; i < inner; ++i) {
      sh.extent[i] = shape[i];
      sh.src_stride[i] = ss[i] * elemSize;
      sh.dst_stride[i] = ds[i] * elemSize;
    }
    sh.extent[inner] = run_bytes / unit;
    sh.src_stride[inner] = sh.dst_stride[inner] = unit;
    int64_t units = total / run * sh.extent[inner];
    DeviceState *st = device_state();
    if (!st)
      return MTRT_RUNTIME_ERROR;
    const int64_t blocks = std::min<int64_t>((units + 255) / 256, int64_t(num_compute_units(st)) * 32);
    KernelName name("mtrt_copy_strided_b");
    name + int(unit);
    void *args[] = {&sbase, &dbase, &units, &krank, &sh};
    return launch(st, name, uint32_t(blocks), 256, hs, args);
  }

  // Ordinary host memory on one side (or more dimensions than the kernel takes): one copy per contiguous run.
  std::vector<int64_t> idx(size_t(inner), 0);
  for (;;) {
    int64_t so = 0, dof = 0;
    for (int64_t i = 0; i < inner; ++i) {
      so += idx[size_t(i)] * ss[i];
      dof += idx[size_t(i)] * ds[i];
    }
    RETURN_IF_RT(hipMemcpyAsync(dbase + dof * elemSize, sbase + so * elemSize, size_t(run * elemSize), hipMemcpyDefault, hs));
    int64_t d = inner - 1;
    while (d >= 0 && ++idx[size_t(d)] == shape[d])
      idx[size_t(d--)] = 0;
    if (d < 0)
      break;
  }
  return MTRT_OK;
}

int32_t mtrt_lua_cuda_get_active_device(int32_t *out_device) {
  if (!out_device)
    return set_error(MTRT_INVALID_ARGUMENT, "out_device must not be null");
  int device = 0;
  *out_device = 0;
  RETURN_IF_RT(hipGetDevice(&device));
  *out_device = device;
  return MTRT_OK;
}

int32_t mtrt_lua_cuda_set_active_device(int32_t deviceNumber) {
  RETURN_IF_RT(hipSetDevice(deviceNumber));
  return MTRT_OK;
}

int32_t mtrt_lua_cuda_get_device(int32_t deviceNumber, int32_t *out_device) {
  // The reference registers this name twice; the later lambda wins and returns the CURRENT device whatever the
  // argument (CUDAModule.cpp:261-267 over :92-97).  Kept as it behaves.
  (void)deviceNumber;
  return mtrt_lua_cuda_get_active_device(out_device);
}

int32_t mtrt_lua_cuda_num_devices(int32_t *out_count) {
  if (!out_count)
    return set_error(MTRT_INVALID_ARGUMENT, "out_count must not be null");
  int n = 0;
  *out_count = 0;
  RETURN_IF_RT(hipGetDeviceCount(&n));
  *out_count = n;
  return MTRT_OK;
}

int32_t mtrt_lua_cuda_get_program_device(int32_t logicalId, int32_t *out_device) {
  if (!out_device)
    return set_error(MTRT_INVALID_ARGUMENT, "out_device must not be null");
  *out_device = 0;
  // One device per program here; the reference indexes its logical-to-ordinal map and reports
  // an out-of-range id the same way (CUDAModule.cpp:560-571).
  if (logicalId != 0)
    return set_error(MTRT_INTERNAL_ERROR,
                     "logical device ID %d is out of range, the number of per-program devices is 1", logicalId);
  int device = 0;
  RETURN_IF_RT(hipGetDevice(&device));
  *out_device = device;
  return MTRT_OK;
}

const struct mtrt_lua_builtin *mtrt_lua_cuda_builtins(size_t *count) {
  static const mtrt_lua_builtin table[] = {
      {"__cuda_load_module", "mtrt_lua_cuda_load_module"},
      {"__cuda_get_function", "mtrt_lua_cuda_get_function"},
      {"__cuda_launch", "mtrt_lua_cuda_launch"},
      {"__cuda_stream_create", "mtrt_lua_cuda_stream_create"},
      {"__cuda_stream_sync", "mtrt_lua_cuda_stream_sync"},
      {"__cuda_stream_destroy", "mtrt_lua_cuda_stream_destroy"},
      {"__cuda_alloc_device", "mtrt_lua_cuda_alloc_device"},
      {"__cuda_free_device", "mtrt_lua_cuda_free_device"},
      {"__cuda_memcpy_host2device", "mtrt_lua_cuda_memcpy"},
      {"__cuda_memcpy_device2host", "mtrt_lua_cuda_memcpy"},
      {"__cuda_memcpy_device2device", "mtrt_lua_cuda_memcpy"},
      {"__cuda_memcpy_host_pinned2device", "mtrt_lua_cuda_memcpy"},
      {"__cuda_memcpy_device2host_pinned", "mtrt_lua_cuda_memcpy"},
      {"__cuda_memset_8", "mtrt_lua_cuda_memset"},
      {"__cuda_memset_16", "mtrt_lua_cuda_memset"},
      {"__cuda_memset_32", "mtrt_lua_cuda_memset"},
      {"__cuda_event_create", "mtrt_lua_cuda_event_create"},
      {"__cuda_event_release", "mtrt_lua_cuda_event_release"},
      {"__cuda_stream_record_event", "mtrt_lua_cuda_stream_record_event"},
      {"__cuda_stream_wait_event", "mtrt_lua_cuda_stream_wait_event"},
      {"__cuda_event_sync", "mtrt_lua_cuda_event_sync"},
      {"__cuda_event_elapsed_msec", "mtrt_lua_cuda_event_elapsed_msec"},
      {"__cuda_alloc_host_pinned", "mtrt_lua_cuda_alloc_host_pinned"},
      {"__cuda_free_host_pinned", "mtrt_lua_cuda_free_host_pinned"},
      {"__cuda_memcpy_strided_async_device2device", "mtrt_lua_cuda_memcpy_strided"},
      {"__cuda_memcpy_strided_async_device2host", "mtrt_lua_cuda_memcpy_strided"},
      {"__cuda_memcpy_strided_async_host2device", "mtrt_lua_cuda_memcpy_strided"},
      {"__cuda_memcpy_strided_async_host_pinned2device", "mtrt_lua_cuda_memcpy_strided"},
      {"__cuda_memcpy_strided_async_device2host_pinned", "mtrt_lua_cuda_memcpy_strided"},
      {"__cuda_num_devices", "mtrt_lua_cuda_num_devices"},
      {"__cuda_get_active_device", "mtrt_lua_cuda_get_active_device"},
      {"__cuda_set_active_device", "mtrt_lua_cuda_set_active_device"},
      {"__cuda_get_device", "mtrt_lua_cuda_get_device"},
      {"__cuda_get_program_device", "mtrt_lua_cuda_get_program_device"},
  };
  if (count)
    *count = sizeof(table) / sizeof(table[0]);
  return table;
}

} // extern "C"
