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
