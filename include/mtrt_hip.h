/* C ABI of libmtrt_hip.so — the MI355X (gfx950) replacement for the executor
 * runtime's CUDA kernel-launch layer plus the hand-written kernel clusters that
 * stand in for the reference's generated PTX.
 *
 * Part 1 keeps the reference's symbol names, argument order and argument widths,
 * so host code emitted by the reference compiler for its C backend links against
 * this library unchanged; handles are opaque pointers (the reference's CUmodule,
 * CUfunction, CUstream and cudaEvent_t are pointers too).  Where the reference
 * takes PTX text these entry points take a gfx950 code object (the output of
 * `hipcc --genco --offload-arch=gfx950`, bundled or bare): there is no JIT step.
 * As in the reference, every failure in part 1 is fatal: the message is printed
 * to stderr as "<file>#<line>: <text>" and the process aborts
 * (mlir-tensorrt/executor/lib/Runtime/Backend/C/CUDAModule.cpp:27-53).
 *
 * Part 2 is the cluster layer: one entry point per kernel cluster of the
 * quantization hot path.  The reference has no such functions — its compiler
 * picks a grid and block for each generated kernel and emits a
 * get-function + launch pair (mlir-tensorrt/compiler/lib/Passes/1_Core/KernelToCUDA/
 * KernelToCUDA.cpp:151-186); these entry points are that emitted code written by
 * hand for the hand-written kernels: they validate shapes and alignment, pick the
 * kernel variant and launch shape for gfx950, build the void** argument array in
 * the reference's device ABI (bare pointers, 64-bit sizes, scalars by value:
 * mlir-tensorrt/kernel/lib/Kernel/Transforms/ExpandMemRefArgs.cpp:65-120) and go
 * through the same module / function / launch path as part 1.  They return a
 * status (0 = ok, codes as mlir-tensorrt/executor/lib/Runtime/StandaloneCPP/
 * MTRTRuntimeStatus.h:31-41) and leave a message for mtrt_hip_last_error().
 * All pointers are device pointers unless stated; nothing is synchronised: work
 * is enqueued on `stream` (NULL = the default stream).
 */
#ifndef MTRT_HIP_H
#define MTRT_HIP_H

#include <stddef.h>
#include <stdint.h>

#define MTRT_CAPI_EXPORTED __attribute__((visibility("default")))

#ifdef __cplusplus
extern "C" {
#endif

typedef struct mtrt_opaque_module *mtrt_module_t;     /* hipModule_t   (reference: CUmodule)    */
typedef struct mtrt_opaque_function *mtrt_function_t; /* hipFunction_t (reference: CUfunction)  */
typedef struct mtrt_opaque_stream *mtrt_stream_t;     /* hipStream_t   (reference: CUstream)    */
typedef struct mtrt_opaque_event *mtrt_event_t;       /* hipEvent_t    (reference: cudaEvent_t) */

/* ------------------------------------------------------------------------- */
/* Part 1 — launch ABI, same names as the reference C backend                  */
/* (mlir-tensorrt/executor/lib/Runtime/Backend/C/CUDAModule.h:55-123)          */
/* ------------------------------------------------------------------------- */

/* CUDAModule.h:55-59 */
MTRT_CAPI_EXPORTED int32_t mtrt_cuda_get_active_device(void);
MTRT_CAPI_EXPORTED int32_t mtrt_cuda_set_active_device(int32_t device);
MTRT_CAPI_EXPORTED int32_t mtrt_cuda_get_device(int32_t device);
/* Called by the LLVM lowering of cuda.num_devices (CUDAToLLVM.cpp:155-156) but neither declared nor
 * defined by the reference's C backend; defined here so that such programs link.  The lowering's other
 * orphan, mtrt_cuda_memcpy_strided_async(stream, rank, descriptor, rank, descriptor) (CUDAToLLVM.cpp:143-150,
 * 502-513), is NOT provided: the call carries no element size, so the bytes to move are not determined. */
MTRT_CAPI_EXPORTED int32_t mtrt_cuda_get_device_count(void);

/* CUDAModule.h:61-65.  The reference header declares stream_create without a
 * parameter while its LLVM lowering passes an i32 device
 * (mlir-tensorrt/compiler/lib/Passes/2_Host/HostToLLVM/CUDAToLLVM/CUDAToLLVM.cpp:67-68);
 * under the SysV x86-64 ABI an ignored integer argument is harmless, so the
 * header form is kept. */
MTRT_CAPI_EXPORTED mtrt_stream_t mtrt_cuda_stream_create(void);
MTRT_CAPI_EXPORTED void mtrt_cuda_stream_destroy(mtrt_stream_t stream);
MTRT_CAPI_EXPORTED void mtrt_cuda_stream_sync(mtrt_stream_t stream);

/* CUDAModule.h:71-85 */
MTRT_CAPI_EXPORTED mtrt_event_t mtrt_cuda_event_create(int32_t device);
MTRT_CAPI_EXPORTED void mtrt_cuda_event_release(mtrt_event_t event);
MTRT_CAPI_EXPORTED void mtrt_cuda_stream_record_event(mtrt_stream_t stream, mtrt_event_t event);
MTRT_CAPI_EXPORTED void mtrt_cuda_stream_wait_event(mtrt_stream_t stream, mtrt_event_t event);
MTRT_CAPI_EXPORTED void mtrt_cuda_event_sync(mtrt_event_t event);
MTRT_CAPI_EXPORTED float mtrt_cuda_event_elapsed_msec(mtrt_event_t start, mtrt_event_t end);

/* CUDAModule.h:87-96.  Pinned or managed requests return host-coherent memory
 * (the reference returns cudaMallocManaged memory for both); device requests
 * are stream-ordered allocations. */
MTRT_CAPI_EXPORTED void *mtrt_cuda_alloc_async(mtrt_stream_t stream, int64_t size, int32_t alignment,
                                               int8_t isHostPinned, int8_t isManaged);
MTRT_CAPI_EXPORTED void mtrt_cuda_memcpy_async(mtrt_stream_t stream, void *src, void *dest,
                                               int64_t size);
MTRT_CAPI_EXPORTED void mtrt_cuda_free(mtrt_stream_t stream, void *ptr, int8_t isHostPinned,
                                       int8_t isManaged);

/* CUDAModule.h:98-102.  `ptxData`/`ptxLen` hold a gfx950 code object, not PTX. */
MTRT_CAPI_EXPORTED mtrt_module_t mtrt_cuda_module_load_from_ptx(const char *ptxData, size_t ptxLen);
MTRT_CAPI_EXPORTED mtrt_module_t mtrt_cuda_module_load_from_ptx_file(const char *filename,
                                                                     size_t filenameLength);
/* CUDAModule.h:104 */
MTRT_CAPI_EXPORTED void mtrt_cuda_module_unload(mtrt_module_t module);
/* CUDAModule.h:106-108.  `name` is NOT NUL-terminated; `length` bytes are used. */
MTRT_CAPI_EXPORTED mtrt_function_t mtrt_cuda_module_get_function(mtrt_module_t module,
                                                                 const char *name, int64_t length);
/* CUDAModule.h:110-115.  args[i] points at the storage of the i-th kernel
 * operand (the driver's kernelParams convention); valid only during the call. */
MTRT_CAPI_EXPORTED void mtrt_cuda_launch_kernel(mtrt_function_t func, int32_t gridX, int32_t gridY,
                                                int32_t gridZ, int32_t blockX, int32_t blockY,
                                                int32_t blockZ, int32_t dynamicSharedMemory,
                                                mtrt_stream_t stream, void **args);
/* CUDAModule.h:117-119 */
MTRT_CAPI_EXPORTED int32_t mtrt_cuda_get_current_device(void);
MTRT_CAPI_EXPORTED int32_t mtrt_cuda_get_program_device(int32_t logicalId);

/* CUDAModule.h:130-205: the type-erased `<name>_cwrapper` twins that emitted C/C++ calls (every handle
 * travels as `void *`).  Header-only, as in the reference; each one forwards to the entry point above. */
#define MTRT_HANDLE(type, p) ((type)(p))
static inline void *mtrt_cuda_stream_create_cwrapper(void) { return (void *)mtrt_cuda_stream_create(); }
static inline void mtrt_cuda_stream_destroy_cwrapper(void *stream) {
  mtrt_cuda_stream_destroy(MTRT_HANDLE(mtrt_stream_t, stream));
}
static inline void mtrt_cuda_stream_sync_cwrapper(void *stream) { mtrt_cuda_stream_sync(MTRT_HANDLE(mtrt_stream_t, stream)); }
static inline void *mtrt_cuda_event_create_cwrapper(int32_t device) { return (void *)mtrt_cuda_event_create(device); }
static inline void mtrt_cuda_event_release_cwrapper(void *event) { mtrt_cuda_event_release(MTRT_HANDLE(mtrt_event_t, event)); }
static inline void mtrt_cuda_stream_record_event_cwrapper(void *stream, void *event) {
  mtrt_cuda_stream_record_event(MTRT_HANDLE(mtrt_stream_t, stream), MTRT_HANDLE(mtrt_event_t, event));
}
static inline void mtrt_cuda_stream_wait_event_cwrapper(void *stream, void *event) {
  mtrt_cuda_stream_wait_event(MTRT_HANDLE(mtrt_stream_t, stream), MTRT_HANDLE(mtrt_event_t, event));
}
static inline void mtrt_cuda_event_sync_cwrapper(void *event) { mtrt_cuda_event_sync(MTRT_HANDLE(mtrt_event_t, event)); }
static inline float mtrt_cuda_event_elapsed_msec_cwrapper(void *start, void *end) {
  return mtrt_cuda_event_elapsed_msec(MTRT_HANDLE(mtrt_event_t, start), MTRT_HANDLE(mtrt_event_t, end));
}
static inline void *mtrt_cuda_alloc_async_cwrapper(void *stream, int64_t size, int32_t alignment, int8_t isHostPinned,
                                                   int8_t isManaged) {
  return mtrt_cuda_alloc_async(MTRT_HANDLE(mtrt_stream_t, stream), size, alignment, isHostPinned, isManaged);
}
static inline void mtrt_cuda_memcpy_async_cwrapper(void *stream, void *src, void *dest, int64_t size) {
  mtrt_cuda_memcpy_async(MTRT_HANDLE(mtrt_stream_t, stream), src, dest, size);
}
static inline void mtrt_cuda_free_cwrapper(void *stream, void *ptr, int8_t isHostPinned, int8_t isManaged) {
  mtrt_cuda_free(MTRT_HANDLE(mtrt_stream_t, stream), ptr, isHostPinned, isManaged);
}
static inline void *mtrt_cuda_module_load_from_ptx_cwrapper(void *ptxData, size_t ptxLen) {
  return (void *)mtrt_cuda_module_load_from_ptx((const char *)ptxData, ptxLen);
}
static inline void *mtrt_cuda_module_load_from_ptx_file_cwrapper(void *filename, size_t filenameLength) {
  return (void *)mtrt_cuda_module_load_from_ptx_file((const char *)filename, filenameLength);
}
static inline void mtrt_cuda_module_unload_cwrapper(void *module) { mtrt_cuda_module_unload(MTRT_HANDLE(mtrt_module_t, module)); }
static inline void *mtrt_cuda_module_get_function_cwrapper(void *module, void *name, int64_t length) {
  return (void *)mtrt_cuda_module_get_function(MTRT_HANDLE(mtrt_module_t, module), (const char *)name, length);
}
static inline void mtrt_cuda_launch_kernel_cwrapper(void *func, int32_t gridX, int32_t gridY, int32_t gridZ, int32_t blockX,
                                                    int32_t blockY, int32_t blockZ, int32_t dynamicSharedMemory,
                                                    void *stream, void *args) {
  mtrt_cuda_launch_kernel(MTRT_HANDLE(mtrt_function_t, func), gridX, gridY, gridZ, blockX, blockY, blockZ,
                          dynamicSharedMemory, MTRT_HANDLE(mtrt_stream_t, stream), (void **)args);
}
static inline int32_t mtrt_cuda_get_current_device_cwrapper(void) { return mtrt_cuda_get_current_device(); }
#undef MTRT_HANDLE

/* ------------------------------------------------------------------------- */
/* Part 2 — kernel clusters of the quantization hot path                       */
/* ------------------------------------------------------------------------- */

/* element types */
enum mtrt_hip_dtype {
  MTRT_F32 = 0,
  MTRT_F16 = 1,
  MTRT_BF16 = 2,
  MTRT_I8 = 3,
  MTRT_F8E4M3FN = 4,
  MTRT_I4 = 5,        /* one int4 per byte, low nibble: the executor's host/buffer storage
                         (mlir-tensorrt/executor/lib/Runtime/Backend/Common/DataTypes.cpp:494-519) */
  MTRT_I4_PACKED = 6, /* two per byte, element 2i in the low nibble: what the reference hands to
                         TensorRT (mlir-tensorrt/tensorrt/lib/Target/TensorRTEncodingOpInterface/
                         NetworkEncoder.cpp:552-595) */
  MTRT_F4_PACKED = 8  /* f4E2M1FN (0, 0.5, 1, 1.5, 2, 3, 4, 6 and a sign), two per byte, element 2i in
                         the low nibble; the block modes of quantize / dequantize allow it
                         (TensorRTOps.td:3133-3194).  Converted through f16 as the reference does
                         (mlir-tensorrt/executor/lib/Passes/ExpandOps.cpp:471-694); 7 is unused */
};

/* how `scale` is addressed; the data tensor is viewed as row-major [d0, d1] */
enum mtrt_hip_scale_kind {
  MTRT_SCALE_UNIFORM = 0, /* per-tensor: scale[0]; `nb` ignored                             */
  MTRT_SCALE_ROW = 1,     /* scale[row % nb]: per-channel on a non-last axis (d0 = outer*C,
                             nb = C) or blocks along the last axis (d1 = block, nb = d0)    */
  MTRT_SCALE_COL = 2      /* scale[(row / nb) * d1 + col]: per-channel on the last axis
                             (nb = d0) or blocks of nb rows along axis 0                    */
};

enum mtrt_hip_flags {
  MTRT_Q_ROUND_TO_INT = 1, /* f8 target: apply round_nearest_even before the clamp, the form
                              StablehloRaiseQDQ.cpp:233-265 matches; integer targets always round */
  MTRT_F8_REFHOST = 2,     /* f8 target: reproduce the reference HOST class bit for bit
                              (DataTypes.cpp:43-122) instead of IEEE RNE + saturate           */
  MTRT_F8_VIA_F16 = 4      /* f8 target: convert f32 -> f16 -> f8, rounding to nearest even TWICE, which is
                              what the reference's generated GPU kernels do
                              (mlir-tensorrt/kernel/lib/Kernel/Transforms/NormalizeQuantizedConversions.cpp:38-118).
                              Differs from the single rounding of the default where the f16 rounding lands on
                              an f8 midpoint (about one input in 250 on normally distributed data).  Not
                              combinable with MTRT_F8_REFHOST.                                 */
};

/* status codes, MTRTRuntimeStatus.h:31-41 */
enum mtrt_hip_status {
  MTRT_OK = 0,
  MTRT_INVALID_ARGUMENT = 1,
  MTRT_NOT_FOUND = 2,
  MTRT_IO_ERROR = 3,
  MTRT_DRIVER_ERROR = 4,
  MTRT_RUNTIME_ERROR = 5,
  MTRT_INTERNAL_ERROR = 7,
  MTRT_UNIMPLEMENTED = 8
};

/* Thread-local message of the most recent failed part-2 call on this thread
 * (MTRTRuntimeStatus.h:48-53 convention); "" if none. */
MTRT_CAPI_EXPORTED const char *mtrt_hip_last_error(void);

/* Loads the built-in kernel module on the current device (idempotent; every
 * part-2 entry point does it on first use).  Fails with MTRT_RUNTIME_ERROR when
 * there is no usable gfx950 device: there is no CPU fallback. */
MTRT_CAPI_EXPORTED int32_t mtrt_hip_init(void);
/* The built-in module, for callers that launch its kernels themselves through
 * mtrt_cuda_module_get_function + mtrt_cuda_launch_kernel.  NULL on failure. */
MTRT_CAPI_EXPORTED mtrt_module_t mtrt_hip_builtin_module(void);
/* The code object bytes of the built-in module (what a reference executable
 * would carry in the data segment that holds PTX today:
 * mlir-tensorrt/compiler/lib/Passes/2_Host/HostToExecutor/CUDAToExecutor/CUDAToExecutor.cpp:858-866). */
MTRT_CAPI_EXPORTED const char *mtrt_hip_builtin_code_object(size_t *size);

/* {abs, reduce-max} cluster + scale = amax / qmax (one f32 divide).
 * Either output may be NULL.  Replaces the generated reduction kernel of
 * mlir-tensorrt/kernel/lib/Kernel/TransformSchedules/FallbackSchedule.cpp:147-343. */
MTRT_CAPI_EXPORTED int32_t mtrt_hip_amax(mtrt_stream_t stream, const void *x, int32_t dtype,
                                         int64_t n, float qmax, float *amax_out, float *scale_out);

/* amax and scale for every scale element of a per-channel or block-wise quantization: the tensor is viewed as
 * [d0, d1] and `scale_kind` / `nb` address the scales exactly as in mtrt_hip_quantize below; each scale element
 * gets amax = max |f32(x)| over the elements that address it and scale = amax / qmax
 * (tripy/examples/nanogpt/weight_loader.py:67-68, 102-115).  MTRT_SCALE_ROW with nb = d0 gives one scale per row
 * (per-token activation scales, per-output-channel weight scales); MTRT_SCALE_COL with nb = 128 the [d0 / 128, d1]
 * scales of int4 block quantization along axis 0; MTRT_SCALE_UNIFORM forwards to mtrt_hip_amax.  Outputs hold nb
 * (row kind) or (d0 / nb) * d1 (col kind) f32 values; either may be NULL. */
MTRT_CAPI_EXPORTED int32_t mtrt_hip_amax_scales(mtrt_stream_t stream, const void *x, int32_t dtype,
                                                int32_t scale_kind, int64_t d0, int64_t d1, int64_t nb,
                                                float qmax, float *amax_out, float *scale_out);

/* Grid reductions (mtrt_hip_amax and the kernels that fold an amax into another pass) meet in a small
 * block of device memory that the library keeps per stream and that every launch leaves zeroed.  A launch
 * that did not run to completion (a device fault, a killed process sharing the context) can leave it
 * non-zero; this call clears the block of `stream` in stream order.  Blocks are also cleared when first
 * bound to a stream and return to the pool when the stream is destroyed through any of the stream-destroy
 * entry points of this library. */
MTRT_CAPI_EXPORTED int32_t mtrt_hip_reset_reductions(mtrt_stream_t stream);

/* mtrt_hip_amax for callers that cannot allocate device memory (code under stream capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same operands and
 * results as mtrt_hip_amax; the reduction's scratch block (5 KiB) is a device array inside this library,
 * one copy per GPU, cleared by a small fill kernel at the start of each call.  The call itself allocates
 * nothing, but mtrt_hip_init() must have run on the current device before (it loads the kernels and looks
 * the array's address up); otherwise MTRT_RUNTIME_ERROR.  n above MTRT_HIP_AMAX_NO_ALLOC_MAX_ELEMENTS
 * is MTRT_INVALID_ARGUMENT.  All calls on one GPU share the block: calls that overlap in time on one GPU
 * (different streams) race; serialise them. */
#define MTRT_HIP_AMAX_NO_ALLOC_MAX_ELEMENTS ((int64_t)1 << 36)
MTRT_CAPI_EXPORTED int32_t mtrt_hip_amax_no_alloc(mtrt_stream_t stream, const void *x, int32_t dtype,
                                                  int64_t n, float qmax, float *amax_out,
                                                  float *scale_out);

/* tensorrt.quantize semantics (TensorRTOps.td:3133-3194) in the StableHLO form
 * of StablehloRaiseQDQ.cpp:233-265: q = convert(clamp(lo, rne(f32(x) / scale), hi)).
 * x_dtype in {F32,F16,BF16}; q_dtype in {I8,F8E4M3FN,I4,I4_PACKED,F4_PACKED}; scale is f32. */
MTRT_CAPI_EXPORTED int32_t mtrt_hip_quantize(mtrt_stream_t stream, const void *x, int32_t x_dtype,
                                             void *q, int32_t q_dtype, const float *scale,
                                             int32_t scale_kind, int64_t d0, int64_t d1, int64_t nb,
                                             int32_t flags);
/* tensorrt.dequantize semantics (TensorRTOps.td:3408-3445; StablehloRaiseQDQ.cpp:407-418):
 * y = narrow(f32(q) * scale). */
MTRT_CAPI_EXPORTED int32_t mtrt_hip_dequantize(mtrt_stream_t stream, const void *q, int32_t q_dtype,
                                               void *y, int32_t y_dtype, const float *scale,
                                               int32_t scale_kind, int64_t d0, int64_t d1,
                                               int64_t nb);
/* quantize followed by dequantize in one pass over x (the fake-quant pair of
 * tripy/nvtripy/frontend/module/linear.py:112-151); writes q and y (same type as x). */
MTRT_CAPI_EXPORTED int32_t mtrt_hip_quantize_dequantize(mtrt_stream_t stream, const void *x,
                                                        int32_t x_dtype, void *q, int32_t q_dtype,
                                                        void *y, const float *scale,
                                                        int32_t scale_kind, int64_t d0, int64_t d1,
                                                        int64_t nb, int32_t flags);

/* Dynamic per-tensor quantization, the whole chain of a dynamic-scale Q/DQ in one call:
 *   amax = max |f32(x)| ; scale = amax / qmax ; q = convert(clamp(rne?(f32(x) / scale))) ; y = narrow(f32(q) * scale)
 * (clusters of KernelSegmentation.cpp:53-113 in the program form of StablehloRaiseQDQ.cpp:233-265, 407-418; scale rule
 * tripy/examples/nanogpt/weight_loader.py:67-68).  q_dtype: MTRT_I8 or MTRT_F8E4M3FN; y may be NULL (codes only);
 * amax_out may be NULL; scale_out must be given.  Results are bit-identical to mtrt_hip_amax followed by
 * mtrt_hip_quantize_dequantize.  A tensor that fits in the registers of one grid (n / 4 (f32) or n / 8 (f16, bf16)
 * at most 16384 per compute unit, n a multiple of that vector length, x and y 16-byte aligned) runs as ONE
 * launch that reads x once; its workgroups wait for each other's maximum with a bounded number of polls and a
 * workgroup that gives up reduces the tensor by itself, so the launch finishes whatever else occupies the device.
 * Larger or unaligned tensors run as the two launches above. */
MTRT_CAPI_EXPORTED int32_t mtrt_hip_dynamic_quantize_dequantize(mtrt_stream_t stream, const void *x,
                                                                int32_t x_dtype, void *q, int32_t q_dtype,
                                                                void *y, int64_t n, float qmax,
                                                                float *amax_out, float *scale_out,
                                                                int32_t flags);
/* Dynamic per-row (per-token) quantization in one call: for every row r of x [rows, d]
 *   amax[r] = max_c |f32(x[r,c])| ; scale[r] = amax[r] / qmax ; q[r,c] = convert(clamp(rne?(f32(x[r,c]) / scale[r])))
 * the single-use elementwise producers pulled into their consumer as the reference's segmentation does
 * (mlir-tensorrt/compiler/lib/Backends/Kernel/KernelSegmentation.cpp:84-100), with the scale rule of
 * tripy/examples/nanogpt/weight_loader.py:67-68, 102-115.  This is what makes the int8 activations and the per-token
 * scales a_scale[m] that mtrt_hip_gemm_w8a8 takes.  q_dtype: MTRT_I8 or MTRT_F8E4M3FN (one code per byte);
 * scale_out: f32 [rows], required; amax_out: f32 [rows] or NULL; flags as for mtrt_hip_quantize.  Results are
 * bit-identical to mtrt_hip_amax_scales(MTRT_SCALE_ROW, nb = rows) followed by mtrt_hip_quantize(MTRT_SCALE_ROW,
 * nb = rows).  Rows of whole 128-bit vectors (d % 4 == 0 for f32, d % 8 == 0 for f16 / bf16, x 16-byte aligned, q
 * aligned to 4 / 8 bytes) of up to 16384 elements (32768 for f16 / bf16 to int8) run as ONE launch that reads x once,
 * the row held in registers between the reduction and the quantization; other shapes run as those two launches. */
MTRT_CAPI_EXPORTED int32_t mtrt_hip_dynamic_quantize_rows(mtrt_stream_t stream, const void *x, int32_t x_dtype,
                                                          void *q, int32_t q_dtype, int64_t rows, int64_t d,
                                                          float qmax, float *amax_out, float *scale_out,
                                                          int32_t flags);
/* Number of polls a workgroup of the one-launch form spends waiting for the grid's maximum before it computes
 * the maximum by itself (default 65536; 0: never wait).  Returns the previous value.  Process-wide. */
MTRT_CAPI_EXPORTED int32_t mtrt_hip_set_wait_limit(int32_t polls);

/* quantize / dequantize on rank-2 VIEWS (slices, transposes, offset sub-tensors): each tensor operand is a base
 * pointer plus (offset, stride0, stride1) in elements, element (r, c) of the [d0, d1] view at
 * base[offset + r * stride0 + c * stride1], which is how the reference hands a dynamic strided memref to a
 * generated kernel (ExpandMemRefArgs.cpp:65-120: base, offset, sizes, strides; order pinned by
 * compiler/test/Passes/1_Core/KernelToCUDA/kernel-to-cuda.mlir:3-48).  The reference passes only the components
 * that are dynamic in the memref type (kernel/test/Kernel/Bufferization/expand-memref-args.mlir:1-22: a static
 * extent, stride or offset is folded into the kernel); the kernels here are the fully dynamic form and take all
 * of them.  Codes are one per byte (MTRT_I8,
 * MTRT_F8E4M3FN, MTRT_I4); the scale is contiguous and addressed by the logical (r, c) as above.  A view may not
 * reach below its base pointer; that it stays inside the allocation is the caller's responsibility, as it is for
 * generated kernels.  Results equal those of the contiguous entry points on a packed copy of the view. */
typedef struct mtrt_hip_view2d {
  int64_t offset, stride0, stride1;
} mtrt_hip_view2d;
MTRT_CAPI_EXPORTED int32_t mtrt_hip_quantize_view(mtrt_stream_t stream, const void *x, int32_t x_dtype,
                                                  const mtrt_hip_view2d *x_view, void *q, int32_t q_dtype,
                                                  const mtrt_hip_view2d *q_view, const float *scale,
                                                  int32_t scale_kind, int64_t d0, int64_t d1, int64_t nb,
                                                  int32_t flags);
MTRT_CAPI_EXPORTED int32_t mtrt_hip_dequantize_view(mtrt_stream_t stream, const void *q, int32_t q_dtype,
                                                    const mtrt_hip_view2d *q_view, void *y, int32_t y_dtype,
                                                    const mtrt_hip_view2d *y_view, const float *scale,
                                                    int32_t scale_kind, int64_t d0, int64_t d1, int64_t nb);

/* NVFP4 block quantization, the two-level scaling of tensorrt.dynamic_quantize (TensorRTOps.td:3279-3358;
 * verifier mlir-tensorrt/tensorrt/lib/TensorRT/IR/Verification.cpp:1271-1290) in the program form of
 * mlir-tensorrt/integrations/PJRT/test/JAX/test_q_dq_nvfp4.py:21-45, over the [d0, d1] view of the tensor
 * (leading axes folded into d0).  block_axis = 1: blocks of 16 along the last axis (d1 % 16 == 0), scales
 * [d0, d1/16]; block_axis = 0: blocks of 16 along the second-to-last axis (its extent % 16 == 0, d1 % 8 == 0
 * for f16/bf16 or % 4 for f32), scales [d0/16, d1].  q = f4E2M1FN codes two per byte over the flattened array
 * (element 2i in the low nibble), scales = one f8E4M3FN byte per block, tensor_amax = device pointer to the
 * f32 amax of the whole tensor (mtrt_hip_amax writes it); the second-level scale of the op is
 * tensor_amax / 2688.  x / y: f32, f16 or bf16, 16-byte aligned; q 16-byte aligned; scales 8-byte aligned.
 * NaN elements and all-zero blocks follow the program (code 0).  A tensor_amax below the largest finite |x|
 * (not what the op computes) lets a block scale exceed the f8 range; the byte stored for such a block is the
 * hardware conversion's and is not specified here. */
MTRT_CAPI_EXPORTED int32_t mtrt_hip_nvfp4_quantize(mtrt_stream_t stream, const void *x, int32_t x_dtype,
                                                   void *q_packed, void *scales, const float *tensor_amax,
                                                   int64_t d0, int64_t d1, int32_t block_axis);
MTRT_CAPI_EXPORTED int32_t mtrt_hip_nvfp4_dequantize(mtrt_stream_t stream, const void *q_packed,
                                                     const void *scales, const float *tensor_amax, void *y,
                                                     int32_t y_dtype, int64_t d0, int64_t d1,
                                                     int32_t block_axis);

/* LayerNorm over the last dimension, one launch
 * (RaiseNormalizations.pdll:277-308; TensorRTOps.td:1303-1373); x, gamma, beta, y share dtype. */
MTRT_CAPI_EXPORTED int32_t mtrt_hip_layernorm(mtrt_stream_t stream, const void *x, const void *gamma,
                                              const void *beta, void *y, int32_t dtype, int64_t rows,
                                              int64_t d, float eps);
/* softmax over the last dimension, one launch (StablehloMatchers.cpp:311-335; TensorRTOps.td:1769-1796) */
MTRT_CAPI_EXPORTED int32_t mtrt_hip_softmax(mtrt_stream_t stream, const void *x, void *y,
                                            int32_t dtype, int64_t rows, int64_t d);

/* W8A8 GEMM with fused dequantize epilogue:
 *   acc[m,n] = sum_k i32(a[m,k]) * i32(w[k,n])   ;   y[m,n] = f16((f32(acc) * a_scale[m]) * w_scale[n])
 * (the int8 form of the quantized Linear of tripy/nvtripy/frontend/module/linear.py:112-151; the
 * reference's code generator emits an FMA loop nest for it, mlir-tensorrt/kernel/test/Kernel/
 * TransformSchedules/fallback-schedule-matmul.mlir:24).  Weights are program constants: they are
 * re-laid ONCE from the program's [K,N] into [N,K] (K contiguous, what the matrix cores read) by
 * the prepack call; the GEMM takes the re-laid weights.  a: int8 [M,K]; a_scale: f32 [M];
 * w_scale: f32 [N]; y: f16 [M,N].  Any M, K, N and any operand alignment run on the matrix cores (K that
 * is a multiple of 128 with 16-byte aligned operands on the faster tile loop; up to 128 rows with weights
 * of moderate size on kernels bound by reading the weights once); the sums are integers, so every kernel
 * gives the same bits. */
MTRT_CAPI_EXPORTED int32_t mtrt_hip_gemm_w8a8_prepack(mtrt_stream_t stream, const void *w_kn,
                                                      void *w_nk, int64_t K, int64_t N);
MTRT_CAPI_EXPORTED int32_t mtrt_hip_gemm_w8a8(mtrt_stream_t stream, const void *a, const void *w_nk,
                                              const float *a_scale, const float *w_scale, void *y,
                                              int64_t M, int64_t K, int64_t N);

/* The same GEMM on the faster kernel that takes the weights from a FRAGMENT-ORDER re-layout straight
 * into registers (the [N,K] form above goes through LDS and is kept for callers that hold the weights
 * in that form only).  `w` is the program's [K,N] constant (w_is_nk = 0) or an [N,K] array (w_is_nk = 1);
 * w_frag holds mtrt_hip_gemm_w8a8_fragments_bytes(K, N) bytes (0 = shape not supported: K % 128 != 0)
 * and must be 16-byte aligned.  Same results, bit for bit.  Up to 32 rows (decode) take a kernel of their own
 * that is bound by reading the weights once, not by a tile's K loop, and so do 33 to 128 rows while that is
 * shorter than a tile launch. */
MTRT_CAPI_EXPORTED int64_t mtrt_hip_gemm_w8a8_fragments_bytes(int64_t K, int64_t N);
MTRT_CAPI_EXPORTED int32_t mtrt_hip_gemm_w8a8_prepack_fragments(mtrt_stream_t stream, const void *w,
                                                                int32_t w_is_nk, void *w_frag, int64_t K,
                                                                int64_t N);
MTRT_CAPI_EXPORTED int32_t mtrt_hip_gemm_w8a8_fragments(mtrt_stream_t stream, const void *a,
                                                        const void *w_frag, const float *a_scale,
                                                        const float *w_scale, void *y, int64_t M, int64_t K,
                                                        int64_t N);

/* W4A16 block-wise GEMM:
 *   wd[k,n] = f16(f16(w[k,n]) * scale[k / block, n])   ;   y[m,n] = f16(sum_k f32(a[m,k]) * f32(wd[k,n]))
 * (weight-only int4 Linear, linear.py:112-151; block dequantize TensorRTOps.td:3408-3445).
 * a: f16 [M,K]; w_kn_packed: int4 [K,N] two per byte over the flattened array, element 2i in the
 * low nibble (NetworkEncoder.cpp:552-595); scale: f16 [K/block, N]; y: f16 [M,N].
 * The matrix-core kernels read the weights from a one-time re-layout (`w_prepacked`, made by the
 * prepack call, mtrt_hip_gemm_w4a16_prepacked_bytes(K, N) bytes, needs K % 64 == 0; it holds the weights in
 * the fragment order of the 32-column kernels and, when K % 128 == 0, once more in the strip order of the
 * M <= 16 kernel, so it is about K * N bytes); they are
 * used when w_prepacked is given and K % 64 == 0, block % 64 == 0, K % block == 0.  Otherwise a
 * matrix-core kernel that dequantises the original nibbles tile by tile reads w_kn_packed directly
 * (any block that divides K, any K and N; several times slower than the re-laid form).  Either weight
 * pointer may be NULL if the other path applies. */
MTRT_CAPI_EXPORTED int64_t mtrt_hip_gemm_w4a16_prepacked_bytes(int64_t K, int64_t N);
MTRT_CAPI_EXPORTED int32_t mtrt_hip_gemm_w4a16_prepack(mtrt_stream_t stream, const void *w_kn_packed,
                                                       void *w_prepacked, int64_t K, int64_t N);
MTRT_CAPI_EXPORTED int32_t mtrt_hip_gemm_w4a16(mtrt_stream_t stream, const void *a,
                                               const void *w_kn_packed, const void *w_prepacked,
                                               const void *scale, void *y, int64_t M, int64_t K,
                                               int64_t N, int64_t block);

/* Dense Linear in one float type: y[m,n] = narrow(sum_k f32(x[m,k]) * f32(w_nk[n,k]) + f32(bias[n])), f32
 * accumulation; bias may be NULL.  The float matmul of the fake-quant Linear (linear.py:112-151:
 * out = x' @ W'^T + b on dequantized operands) for the parameter combinations the two matrix-core clusters
 * above do not express, and of the unquantized module; w_nk is the module's own [out_features, in_features]
 * weight.  The reference generates a tiled FMA loop nest for such a matmul
 * (fallback-schedule-matmul.mlir:24); here every shape with K > 0 runs on the matrix cores (f16 / bf16 / f32
 * MFMA with f32 accumulation), any shape, no alignment needs beyond the element size.  Up to 128 rows with rows
 * in whole 128-byte slices take kernels bound by reading the weights once. */
MTRT_CAPI_EXPORTED int32_t mtrt_hip_linear_dense(mtrt_stream_t stream, const void *x, const void *w_nk,
                                                 const void *bias, void *y, int32_t dtype, int64_t M,
                                                 int64_t K, int64_t N);

/* ------------------------------------------------------------------------- */
/* Part 3 — the interpreter's builtin set, status-returning                    */
/* (mlir-tensorrt/executor/lib/Runtime/Backend/Lua/Modules/CUDA/CUDAModule.cpp) */
/* ------------------------------------------------------------------------- */

/* The reference registers `__cuda_*` builtins in the Lua state as lambdas over the driver API;
 * handles travel as uintptr_t and a failure becomes a Lua error (SET_LUA_ERROR_IF_ERROR).  These
 * are the bodies of those lambdas over HIP: same value conventions (handles as uintptr_t, i32
 * launch dimensions), a status as the return value and mtrt_hip_last_error() as the text a
 * binding raises.  Nothing aborts. */

/* __cuda_load_module(u32 device, uptr data, u64 nbytes) -> uptr (CUDAModule.cpp:297-327).
 * `data` / `nbytes`: a gfx950 code object in host memory (the executable's data segment that
 * holds PTX in the reference); no JIT.  `device` must be the current device. */
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_load_module(uint32_t device, uintptr_t data, uint64_t nbytes,
                                                     uintptr_t *out_module);
/* __cuda_get_function(uptr module, string name) -> uptr (CUDAModule.cpp:287-295); NUL-terminated name. */
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_get_function(uintptr_t module, const char *name,
                                                      uintptr_t *out_function);
/* __cuda_launch(uptr func, i32 grid x,y,z, i32 block x,y,z, i32 smem, uptr stream, uptr argPtrArray)
 * (CUDAModule.cpp:329-342).  The reference asserts func, stream and the argument array non-null;
 * here a null func or argument array is MTRT_INVALID_ARGUMENT and a null stream is the default stream. */
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_launch(uintptr_t func, int32_t gridX, int32_t gridY, int32_t gridZ,
                                                int32_t blockX, int32_t blockY, int32_t blockZ,
                                                int32_t dynamicSharedMemory, uintptr_t stream,
                                                uintptr_t argPtrArray);
/* __cuda_stream_create / _sync / _destroy (CUDAModule.cpp:269-285) */
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_stream_create(uintptr_t *out_stream);
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_stream_sync(uintptr_t stream);
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_stream_destroy(uintptr_t stream);
/* __cuda_alloc_device(stream, nbytes) / __cuda_free_device (CUDAModule.cpp:344-352, 413-421) */
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_alloc_device(uintptr_t stream, uint64_t nbytes, uintptr_t *out_ptr);
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_free_device(uintptr_t stream, uintptr_t ptr);
/* __cuda_memcpy_{host2device,device2host,device2device}(stream, src, srcOffset, dst, dstOffset, nbytes)
 * (CUDAModule.cpp:423-549): one entry point, the direction is found from the pointers. */
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_memcpy(uintptr_t stream, uintptr_t src, uint64_t srcOffset,
                                                uintptr_t dst, uint64_t dstOffset, uint64_t nbytes);
/* __cuda_memset_{8,16,32}(ptr, offset, nbytes, fill) (CUDAModule.cpp:170-205); width in {1,2,4}, runs a
 * fill kernel on `stream` (no memset node, so it can be captured into a graph). */
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_memset(uintptr_t stream, uintptr_t ptr, uint64_t offset,
                                                uint64_t nbytes, uint32_t fill, int32_t width);
/* __cuda_event_create(device) / _release / __cuda_stream_record_event / __cuda_stream_wait_event /
 * __cuda_event_sync / __cuda_event_elapsed_msec (CUDAModule.cpp:112-155).  As in the reference events come
 * from a per-device pool (mlir-tensorrt/executor/lib/Runtime/Support/CUDAEventPool.cpp): release returns the
 * event to the pool, the next create on that device reuses it. */
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_event_create(int32_t device, uintptr_t *out_event);
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_event_release(uintptr_t event);
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_stream_record_event(uintptr_t stream, uintptr_t event);
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_stream_wait_event(uintptr_t stream, uintptr_t event);
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_event_sync(uintptr_t event);
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_event_elapsed_msec(uintptr_t start, uintptr_t end, float *out_ms);
/* __cuda_alloc_host_pinned(nbytes, alignment) / __cuda_free_host_pinned(stream, ptr) (CUDAModule.cpp:354-376,
 * 400-411).  Pinned memory is allocated, never registered.  The free is ordered after the work already queued
 * on `stream` (the reference's PinnedMemoryAllocator::freeAsync): the block is released once the stream has
 * passed that point, at the latest by a later alloc / free call or at process exit. */
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_alloc_host_pinned(uint64_t nbytes, int32_t alignment, uintptr_t *out_ptr);
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_free_host_pinned(uintptr_t stream, uintptr_t ptr);
/* __cuda_memcpy_strided_async_{device2device,device2host,host2device}(stream, rank, elemSize, src, srcOffset,
 * srcShapeAndStrides, dst, dstOffset, dstShapeAndStrides) (CUDAModule.cpp:210-255): shapes then strides, in
 * elements, `rank` values each; the offsets are memref offsets, in ELEMENTS as well (the copy starts at
 * pointer + offset * elemSize, mlir-tensorrt/executor/lib/Support/StridedCopy.cpp:37-38).  When the device can
 * address both views (device memory, pinned or managed host memory; up to 7 dimensions that are not dense on both
 * sides) one kernel walks the index space, moving units of up to 16 bytes; otherwise (ordinary host memory on one
 * side) the copy is issued run by contiguous run.  The reference issues one copy per element (StridedCopy.cpp:57-75). */
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_memcpy_strided(uintptr_t stream, int64_t rank, int64_t elemSize,
                                                        uintptr_t src, uint64_t srcOffset,
                                                        const int64_t *srcShapeAndStrides, uintptr_t dst,
                                                        uint64_t dstOffset, const int64_t *dstShapeAndStrides);
/* __cuda_get_active_device / __cuda_set_active_device (CUDAModule.cpp:99-107) and __cuda_get_device(deviceNumber):
 * the reference registers that last name twice and the later lambda (CUDAModule.cpp:261-267) returns the current
 * device whatever the argument; so does this one. */
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_get_active_device(int32_t *out_device);
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_set_active_device(int32_t deviceNumber);
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_get_device(int32_t deviceNumber, int32_t *out_device);
/* __cuda_num_devices (CUDAModule.cpp:86-90) and __cuda_get_program_device(logicalId) (:560-571) */
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_num_devices(int32_t *out_count);
MTRT_CAPI_EXPORTED int32_t mtrt_lua_cuda_get_program_device(int32_t logicalId, int32_t *out_device);

/* Name table for a binding to register in a loop: Lua builtin name -> entry point of this part. */
struct mtrt_lua_builtin {
  const char *lua_name;
  const char *symbol;
};
MTRT_CAPI_EXPORTED const struct mtrt_lua_builtin *mtrt_lua_cuda_builtins(size_t *count);

/* Name of the kernel that the most recent successful part-2 call on this thread
 * launched last (for profiles and tests). */
MTRT_CAPI_EXPORTED const char *mtrt_hip_last_kernel(void);

#ifdef __cplusplus
}
#endif
#endif /* MTRT_HIP_H */
