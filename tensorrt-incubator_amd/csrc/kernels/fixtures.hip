// HIP rewrites of the two tiny kernels the reference uses to test its launch ABI.
// They exist so that the known answers of those tests can be replayed through
// mtrt_cuda_module_load_from_ptx(_file) / get_function / launch_kernel:
//   binary_shift_right : mlir-tensorrt/compiler/test/IntegrationTests/CUDA/cuda-launch-kernel.mlir:7-45
//                        (memref<1x32x4xi32> in, i32, f32, memref<1x32x4xi32> out; static shapes,
//                         so each memref is one bare pointer)
//   add_kernel         : mlir-tensorrt/compiler/test/IntegrationTests/EmitC/cuda-launch-kernel.ptx:32-37
//                        (in_ptr, out_ptr, u64 offset, u32 n, f32 scalar)
// Built into its own code object (not the built-in module).
#include <hip/hip_runtime.h>
#include <stdint.h>

extern "C" __global__ void binary_shift_right(const int32_t* in, int32_t shift_i, float shift_f_bits, int32_t* out) {
  const uint32_t idx = (blockIdx.x * 32u + threadIdx.x) * 4u;
  // The reference kernel extracts element 0 four times, so all four lanes of the
  // vector receive in[idx] >> shift.
  const uint32_t shift = uint32_t(shift_i) + __float_as_uint(shift_f_bits);
  const uint32_t v = uint32_t(in[idx]) >> shift;
  out[idx] = int32_t(v);
  out[idx + 1] = int32_t(v);
  out[idx + 2] = int32_t(v);
  out[idx + 3] = int32_t(v);
}

extern "C" __global__ void add_kernel(const float* in_ptr, float* out_ptr, uint64_t offset, uint32_t n, float scalar) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const uint64_t idx = offset + uint64_t(i);
  out_ptr[idx] = in_ptr[idx] + scalar;
}
