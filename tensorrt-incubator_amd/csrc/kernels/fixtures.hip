// HIP rewrites of the two tiny kernels the reference uses to test its launch ABI.
// They exist so that the known answers of those tests can be replayed through
// mtrt_cuda_module_load_from_ptx(_file) / get_function / launch_kernel:
//   binary_shift_right : mlir-tensorrt/compiler/test/IntegrationTests/CUDA/cuda-launch-kernel.mlir:7-45
//                        (memref<1x32x4xi32> in, i32, f32, memref<1x32x4xi32> out; static shapes,
//                         so each memref is one bare pointer)
//   add_kernel         : mlir-tensorrt/compiler/test/IntegrationTests/EmitC/cuda-launch-kernel.ptx:32-37
//                        (in_ptr, out_ptr, u64 offset, u32 n, f32 scalar)
// Built into its own code object (not the built-in module), together with the two measurement yardsticks at
// the end of this file: a plain streaming copy and a matrix-core-only loop.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "common.hpp"

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

// ---- measurement yardsticks (benchmark and profiles only; never launched by the library) ------------------------
using namespace mtrt_dev;

// Plain streaming copy, 128 bits per lane per step.  Its HBM traffic is known exactly (n bytes read, n bytes
// written), so hardware byte counters are calibrated against it and the bandwidth of the memory-bound clusters is
// compared with it.
// (src, dst, nvec) ; nvec 128-bit vectors, both pointers 16-byte aligned
extern "C" __global__ void __launch_bounds__(256) mtrt_copy_b128(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                                int64_t nvec) {
  const int64_t stride = int64_t(gridDim.x) * blockDim.x;
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec; i += stride)
    __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

// The two one-directional companions of the copy, one 128-bit access per lane: what the memory system sustains for a
// stream that is only read (the loaded words are folded together and stored only if they equal `key`, which the
// caller picks so that no lane stores) and for a stream that is only written.
// (src, sink, nvec, key) / (dst, nvec, value) ; grid = ceil(nvec / 256), block = 256
extern "C" __global__ void __launch_bounds__(256) mtrt_read_b128(const u32x4* __restrict__ src, uint32_t* __restrict__ sink,
                                                                int64_t nvec, uint32_t key) {
  const int64_t stride = int64_t(gridDim.x) * blockDim.x;
  uint32_t fold = 0;
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec; i += stride) {
    const u32x4 v = __builtin_nontemporal_load(src + i);
    fold |= (v[0] ^ key) & (v[1] ^ key) & (v[2] ^ key) & (v[3] ^ key);
  }
  if (fold == 0xFFFFFFFFu) sink[0] = fold;             // never true for the all-zero key on the benchmark's fill pattern
}
extern "C" __global__ void __launch_bounds__(256) mtrt_fill_b128(u32x4* __restrict__ dst, int64_t nvec, uint32_t value) {
  const int64_t stride = int64_t(gridDim.x) * blockDim.x;
  const u32x4 v = {value, value, value, value};
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec; i += stride)
    __builtin_nontemporal_store(v, dst + i);
}

// Matrix-core yardstick: what MFMA rate does the chip sustain on GIVEN operand data with no
// memory traffic at all?  One wave per SIMD loads eight 16-byte fragments once and then issues
// `ksteps` rounds of 16 independent MFMAs (a 4 x 4 register tile on fixed fragments, nothing else in the
// loop but its counter).  The rate depends on the data: the matrix cores run into the board's power limit and
// the clock drops when the operands toggle (measured on one MI355X: about 82 % of the
// published dense peak on zeros, 53-57 % on random int8 / normally distributed f16), so the
// GEMM kernels are judged against this number as well as against the published one.
// (src: at least 2^24 bytes of operand data, out: gridDim.x * 256 ints, i32 ksteps) ; block = 256.
namespace mfma_probe {
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

#define MTRT_MFMA_PROBE_BODY(ACC_T, ZERO, MFMA)                                                        \
  const int t = threadIdx.x + blockIdx.x * 256;                                                         \
  v4i a[4], b[4];                                                                                       \
  for (int i = 0; i < 4; ++i) {                                                                         \
    a[i] = src[(t * 8 + i) & 0xFFFFF];                                                                  \
    b[i] = src[(t * 8 + 4 + i) & 0xFFFFF];                                                              \
  }                                                                                                     \
  ACC_T acc[4][4];                                                                                      \
  for (int i = 0; i < 4; ++i)                                                                           \
    for (int j = 0; j < 4; ++j)                                                                         \
      for (int r = 0; r < 16; ++r) acc[i][j][r] = ZERO;                                                 \
  for (int it = 0; it < ksteps; ++it) {                                                                 \
    for (int i = 0; i < 4; ++i)                                                                         \
      for (int j = 0; j < 4; ++j) acc[i][j] = MFMA;                                                     \
  }                                                                                                     \
  ACC_T tot = acc[0][0];                                                                                \
  for (int i = 0; i < 4; ++i)                                                                           \
    for (int j = 0; j < 4; ++j)                                                                         \
      if (i + j) tot += acc[i][j];                                                                      \
  int x = 0;                                                                                            \
  for (int r = 0; r < 16; ++r) x += int(tot[r]);                                                        \
  out[t] = x;

extern "C" __global__ void __launch_bounds__(256, 1) mtrt_mfma_probe_f16(const v4i* __restrict__ src, int* __restrict__ out,
                                                                       int ksteps) {
  MTRT_MFMA_PROBE_BODY(v16f, 0.0f,
                       __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a[i]), __builtin_bit_cast(v8h, b[j]), acc[i][j], 0, 0, 0))
}
extern "C" __global__ void __launch_bounds__(256, 1) mtrt_mfma_probe_i8(const v4i* __restrict__ src, int* __restrict__ out,
                                                                      int ksteps) {
  MTRT_MFMA_PROBE_BODY(v16i, 0, __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], acc[i][j], 0, 0, 0))
}
}  // namespace mfma_probe

