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

#include <cstdint>

#include "mtrt_hip.h"

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

/* MTRTRuntimeCuda.h:36-43 */
MTRT_CAPI_EXPORTED Status cuda_get_current_device(int32_t *outDevice);
MTRT_CAPI_EXPORTED Status cuda_get_program_device(int32_t logicalDevice, int32_t *outDevice);
MTRT_CAPI_EXPORTED Status cuda_stream_sync(mtrt_stream_t stream);
/* MTRTRuntimeCuda.h:45-52 */
MTRT_CAPI_EXPORTED Status cuda_alloc(mtrt_stream_t stream, int64_t sizeBytes, bool isPinned, bool isManaged,
                                     void **outPtr);
MTRT_CAPI_EXPORTED Status cuda_free(mtrt_stream_t stream, void *ptr, int8_t isHostPinned, int8_t isManaged);
MTRT_CAPI_EXPORTED Status cuda_copy(mtrt_stream_t stream, void *src, void *dest, int64_t sizeBytes);
/* MTRTRuntimeCuda.h:54-60 */
MTRT_CAPI_EXPORTED Status cuda_module_create_from_ptx_file(const char *filename, mtrt_module_t *outModule);
MTRT_CAPI_EXPORTED Status cuda_module_destroy(mtrt_module_t module);
MTRT_CAPI_EXPORTED Status cuda_module_get_func(mtrt_module_t module, const char *name, mtrt_function_t *outFunc);
/* MTRTRuntimeCuda.h:75-79 */
MTRT_CAPI_EXPORTED Status cuda_launch_kernel(mtrt_function_t func, int32_t gridX, int32_t gridY, int32_t gridZ,
                                             int32_t blockX, int32_t blockY, int32_t blockZ,
                                             int32_t dynamicSharedMemoryBytes, mtrt_stream_t stream,
                                             void **arguments);
/* MTRTRuntimeCuda.h:93-109 */
MTRT_CAPI_EXPORTED Status cuda_event_create(int32_t device, mtrt_event_t *outEvent);
MTRT_CAPI_EXPORTED Status cuda_event_release(mtrt_event_t event);
MTRT_CAPI_EXPORTED Status cuda_stream_record_event(mtrt_stream_t stream, mtrt_event_t event);
MTRT_CAPI_EXPORTED Status cuda_stream_wait_event(mtrt_stream_t stream, mtrt_event_t event);
MTRT_CAPI_EXPORTED Status cuda_event_sync(mtrt_event_t event);
MTRT_CAPI_EXPORTED Status cuda_event_elapsed_msec(mtrt_event_t start, mtrt_event_t end, float *outMs);

} // namespace mtrt

#endif /* MTRT_HIP_STANDALONE_H */
