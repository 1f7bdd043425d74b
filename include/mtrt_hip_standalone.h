/* C++ flavour of the launch layer: the `namespace mtrt` functions that EmitC-generated host code
 * calls in the reference's StandaloneCPP runtime
 * (mlir-tensorrt/executor/lib/Runtime/StandaloneCPP/MTRTRuntimeCuda.h:36-110), over HIP.
 *
 * Same function names, argument order and error behaviour: every function returns a Status
 * (int32_t, 0 = success, codes of MTRTRuntimeStatus.h:31-41), writes its result through an out
 * parameter, rejects null out parameters / empty names with InvalidArgument, and leaves a
 * message for mtrt::get_last_error_message() (thread-local, MTRTRuntimeStatus.h:48-53).
 * Handle types are HIP's (hipModule_t, hipFunction_t, hipStream_t, hipEvent_t are pointers, like
 * CUmodule, CUfunction, CUstream, cudaEvent_t).  `cuda_module_create_from_ptx_file` reads a
 * gfx950 code object file, not PTX.  The functions are exported from libmtrt_hip.so; they share
 * the driver path of the C entry points in mtrt_hip.h.
 */
#ifndef MTRT_HIP_STANDALONE_H
#define MTRT_HIP_STANDALONE_H

#include <array>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <type_traits>
#include <utility>

#include "mtrt_hip.h"

/* Generated EmitC text spells the handle types with their CUDA names
 * (mlir-tensorrt/compiler/lib/Passes/2_Host/HostToEmitC/HostToEmitC.cpp:134-140): the same opaque pointers here.
 * Define MTRT_HIP_NO_CUDA_TYPE_NAMES before including this header if those names are taken. */
#ifndef MTRT_HIP_NO_CUDA_TYPE_NAMES
typedef mtrt_module_t CUmodule;
typedef mtrt_function_t CUfunction;
typedef mtrt_stream_t CUstream;
typedef mtrt_event_t cudaEvent_t;
#endif

namespace mtrt {

/* MTRTRuntimeStatus.h:31-45 */
enum class ErrorCode : int32_t {
  Success = 0,
  InvalidArgument = 1,
  NotFound = 2,
  IOError = 3,
  CUDADriverError = 4,   /* here: an error from the HIP module / launch calls */
  CUDARuntimeError = 5,  /* here: an error from the HIP stream / event / memory calls */
  TensorRTError = 6,
  InternalError = 7,
  Unimplemented = 8,
};
using Status = int32_t;
inline constexpr Status ok() { return 0; }

/* MTRTRuntimeStatus.h:48-53 */
MTRT_CAPI_EXPORTED const char *get_last_error_message();
MTRT_CAPI_EXPORTED void clear_last_error_message();

/* MTRTRuntimeStatus.h:55-66 */
namespace detail {
MTRT_CAPI_EXPORTED void set_last_error_message_v(const char *fmt, va_list ap);
inline void set_last_error_message(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  set_last_error_message_v(fmt, ap);
  va_end(ap);
}
} // namespace detail

/* MTRTRuntimeStatus.h:68 */
inline Status make_status(ErrorCode code) { return static_cast<Status>(code); }

/* MTRTRuntimeStatus.h:70-81: what generated code calls after every runtime call
 * (HostToEmitCPatternsCuda.cpp:39-42): prints the thread's last message and aborts on a non-zero status. */
inline void abort_on_error(Status st) {
  if (st == ok())
    return;
  const char *msg = get_last_error_message();
  if (msg && msg[0] != '\0')
    std::fprintf(stderr, "%s\n", msg);
  std::abort();
}

/* ---- memref descriptors, MTRTRuntimeCore.h:46-214 (header-only there as well) ------------------------- */

/* MTRTRuntimeCore.h:46-59 */
template <class To, class From>
To bit_cast(From src) {
  static_assert(sizeof(To) == sizeof(From) && std::is_trivially_copyable<To>::value &&
                    std::is_trivially_copyable<From>::value,
                "mtrt::bit_cast needs two trivially copyable types of one size");
  To result;                               /* the object representation copied over: defined for any such pair */
  std::memcpy(static_cast<void *>(&result), static_cast<const void *>(&src), sizeof result);
  return result;
}

/* MTRTRuntimeCore.h:67-88: offset, shape and strides count ELEMENTS, not bytes. */
template <unsigned Rank>
struct RankedMemRef {
  void *allocated;
  void *aligned;
  int64_t offset;
  std::array<int64_t, Rank> shape;
  std::array<int64_t, Rank> strides;
};
template <>
struct RankedMemRef<0> {
  void *allocated;
  void *aligned;
  int64_t offset;
};

/* MTRTRuntimeCore.h:96-107: start pointer + shape of a canonically laid out buffer. */
template <unsigned Rank>
struct PtrAndShape {
  void *bufferStart;
  std::array<int64_t, Rank> shape;
};
template <>
struct PtrAndShape<0> {
  void *bufferStart;
};

/* MTRTRuntimeCore.h:113-123 */
struct UnrankedMemRef {
  int64_t rank;
  const void *rankedDescriptor;
};
struct UnrankedMemRefMut {
  int64_t rank;
  void *rankedDescriptor;
};

/* MTRTRuntimeCore.h:126-146 */
template <unsigned Rank>
UnrankedMemRef make_unranked_descriptor(int64_t rank, const RankedMemRef<Rank> &rankedDescriptor) {
  return UnrankedMemRef{rank, static_cast<const void *>(&rankedDescriptor)};
}
template <unsigned Rank>
UnrankedMemRef make_unranked_descriptor(int64_t rank, const PtrAndShape<Rank> &rankedDescriptor) {
  return UnrankedMemRef{rank, static_cast<const void *>(&rankedDescriptor)};
}
inline UnrankedMemRefMut make_unranked_descriptor_mut_ptr(int64_t rank, void *rankedDesc) {
  return UnrankedMemRefMut{rank, rankedDesc};
}

/* MTRTRuntimeCore.h:149-171: (allocated, aligned, offset, shape..., strides...) */
template <unsigned Rank, typename... Args>
auto make_memref_descriptor(void *allocated, void *aligned, int64_t offset, Args &&...args) {
  static_assert(sizeof...(Args) == Rank * 2, "expected 2*Rank arguments: shape..., strides...");
  const std::array<int64_t, Rank * 2> all{static_cast<int64_t>(std::forward<Args>(args))...};
  RankedMemRef<Rank> d{allocated, aligned, offset, {}, {}};
  for (unsigned i = 0; i < Rank; ++i) {
    d.shape[i] = all[i];
    d.strides[i] = all[Rank + i];
  }
  return d;
}
template <>
inline auto make_memref_descriptor<0>(void *allocated, void *aligned, int64_t offset) {
  return RankedMemRef<0>{allocated, aligned, offset};
}

/* MTRTRuntimeCore.h:174-183 */
template <unsigned Rank, typename... Args>
auto make_ptr_shape_descriptor(void *start, Args &&...args) {
  return PtrAndShape<Rank>{start, std::array<int64_t, Rank>{static_cast<int64_t>(std::forward<Args>(args))...}};
}
template <>
inline auto make_ptr_shape_descriptor<0>(void *start) {
  return PtrAndShape<0>{start};
}

/* MTRTRuntimeCore.h:186-214 */
template <typename T>
void *memref_descriptor_get_allocated_ptr(const T &memref) { return memref.allocated; }
template <typename T>
void *memref_descriptor_get_aligned_ptr(const T &memref) { return memref.aligned; }
template <typename T>
int64_t memref_descriptor_get_offset(const T &memref) { return memref.offset; }
template <typename T>
int64_t memref_descriptor_get_dim_size(const T &memref, int32_t dim) { return memref.shape[dim]; }
template <unsigned Rank>
int64_t memref_descriptor_get_stride(const RankedMemRef<Rank> &memref, int32_t dim) { return memref.strides[dim]; }

/* ---- host memory and constants, MTRTRuntimeCore.h:220-236 ---------------------------------------------- */

/* Aligned host allocation (alignment: a power of two; 0 bytes: success, no pointer). */
MTRT_CAPI_EXPORTED Status host_aligned_alloc(int64_t sizeBytes, int32_t alignment, void **outPtr);
MTRT_CAPI_EXPORTED void host_free(void *ptr);
/* Loads a constant blob (the weights of a compiled program) into the memory space `space`
 * (0 unknown / 1 host: aligned host memory; 2 host-pinned; 3 device; 4 unified).  Relative names are looked up
 * under $MTRT_ARTIFACTS_DIR first, then under the working directory; a missing file is NotFound and the message
 * lists what was tried (MTRTRuntimeCore.cpp:76-93, 168-189). */
MTRT_CAPI_EXPORTED Status constant_load_from_file(const char *filename, int32_t align, int32_t space, void **outPtr);
MTRT_CAPI_EXPORTED void constant_destroy(void *data, int32_t space);

/* MTRTRuntimeCuda.h:36-43 */
MTRT_CAPI_EXPORTED Status cuda_get_current_device(int32_t *outDevice);
MTRT_CAPI_EXPORTED Status cuda_get_program_device(int32_t logicalDevice, int32_t *outDevice);
MTRT_CAPI_EXPORTED Status cuda_stream_sync(mtrt_stream_t stream);
/* MTRTRuntimeCuda.h:45-52 */
MTRT_CAPI_EXPORTED Status cuda_alloc(mtrt_stream_t stream, int64_t sizeBytes, bool isPinned, bool isManaged,
                                     void **outPtr);
MTRT_CAPI_EXPORTED Status cuda_free(mtrt_stream_t stream, void *ptr, int8_t isHostPinned, int8_t isManaged);
MTRT_CAPI_EXPORTED Status cuda_copy(mtrt_stream_t stream, void *src, void *dest, int64_t sizeBytes);
/* MTRTRuntimeCuda.h:54-60.  The file holds a gfx950 code object; relative names are looked up under
 * $MTRT_ARTIFACTS_DIR first, then under the working directory; a missing file is NotFound. */
MTRT_CAPI_EXPORTED Status cuda_module_create_from_ptx_file(const char *filename, mtrt_module_t *outModule);
MTRT_CAPI_EXPORTED Status cuda_module_destroy(mtrt_module_t module);
MTRT_CAPI_EXPORTED Status cuda_module_get_func(mtrt_module_t module, const char *name, mtrt_function_t *outFunc);
/* MTRTRuntimeCuda.h:75-79 */
MTRT_CAPI_EXPORTED Status cuda_launch_kernel(mtrt_function_t func, int32_t gridX, int32_t gridY, int32_t gridZ,
                                             int32_t blockX, int32_t blockY, int32_t blockZ,
                                             int32_t dynamicSharedMemoryBytes, mtrt_stream_t stream,
                                             void **arguments);
/* Two names the reference mentions but never defines are NOT provided: cuda_copy_using_descriptor
 * (declared at MTRTRuntimeCuda.h:81-88, defined and called nowhere) and cuda_copy_strided (emitted by
 * HostToEmitCPatternsCuda.cpp:441-444 for strided copies, declared and defined nowhere).  Both receive void
 * pointers and descriptors that count elements, so the element size - and with it the bytes to move - is not
 * part of the call. */

/* MTRTRuntimeCuda.h:93-109 */
MTRT_CAPI_EXPORTED Status cuda_event_create(int32_t device, mtrt_event_t *outEvent);
MTRT_CAPI_EXPORTED Status cuda_event_release(mtrt_event_t event);
MTRT_CAPI_EXPORTED Status cuda_stream_record_event(mtrt_stream_t stream, mtrt_event_t event);
MTRT_CAPI_EXPORTED Status cuda_stream_wait_event(mtrt_stream_t stream, mtrt_event_t event);
MTRT_CAPI_EXPORTED Status cuda_event_sync(mtrt_event_t event);
MTRT_CAPI_EXPORTED Status cuda_event_elapsed_msec(mtrt_event_t start, mtrt_event_t end, float *outMs);

} // namespace mtrt

#endif /* MTRT_HIP_STANDALONE_H */
