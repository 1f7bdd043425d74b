// Plain streaming copy, 128 bits per lane per step.  It is the yardstick of the
// measurements: its HBM traffic is known exactly (n bytes read, n bytes written),
// so hardware byte counters are calibrated against it and the bandwidth of the
// memory-bound clusters is compared with it.
#include "common.hpp"

using namespace mtrt_dev;

// (src, dst, nvec) ; nvec 128-bit vectors, both pointers 16-byte aligned
extern "C" __global__ void __launch_bounds__(256) mtrt_copy_b128(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                                int64_t nvec) {
  const int64_t stride = int64_t(gridDim.x) * blockDim.x;
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec; i += stride)
    __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

// Matrix-core yardstick: what MFMA rate does the chip sustain on GIVEN operand data with no
// memory traffic at all?  One wave per SIMD loads eight 16-byte fragments once and then issues
// `ksteps` rounds of 16 independent MFMAs (a 4 x 4 register tile, the fragments rotated every
// round).  The rate depends on the data: the matrix cores run into the board's power limit and
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
    const v4i t0 = a[0];                                                                                \
    a[0] = a[1]; a[1] = a[2]; a[2] = a[3]; a[3] = t0;                                                   \
    const v4i t1 = b[0];                                                                                \
    b[0] = b[1]; b[1] = b[2]; b[2] = b[3]; b[3] = t1;                                                   \
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

// Fill kernel behind the interpreter's memset builtins (8-, 16- or 32-bit pattern).  A kernel rather
// than a memset node: it can be recorded into a captured graph like any other launch.
// (p, count, fill, width) ; count elements of `width` bytes, p aligned to `width`.
extern "C" __global__ void __launch_bounds__(256) mtrt_fill(uint8_t* __restrict__ p, int64_t count, uint32_t fill, int32_t width) {
  const int64_t stride = int64_t(gridDim.x) * blockDim.x;
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < count; i += stride) {
    if (width == 4)
      reinterpret_cast<uint32_t*>(p)[i] = fill;
    else if (width == 2)
      reinterpret_cast<uint16_t*>(p)[i] = uint16_t(fill);
    else
      p[i] = uint8_t(fill);
  }
}
