// Utility kernels of the built-in module.
#include "common.hpp"

using namespace mtrt_dev;

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

// Strided copy of a rank <= 8 tensor between two views whose memory the device can address: the device-side form of
// the interpreter's strided memcpy builtins (the reference walks the index space on the host and issues one copy per
// ELEMENT, mlir-tensorrt/executor/lib/Support/StridedCopy.cpp:57-75).  The host has already folded the innermost
// dimensions that are dense in both views into the unit that is moved and appended the units of one run as a last
// dimension, so consecutive lanes move consecutive units of a run.  Strides are in BYTES and may be negative.
struct StridedCopyShape {
  int64_t extent[8];
  int64_t src_stride[8];
  int64_t dst_stride[8];
};
template <typename U>
__device__ __forceinline__ void copy_strided(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, int64_t total,
                                             int32_t rank, const StridedCopyShape& sh) {
  const int64_t step = int64_t(gridDim.x) * blockDim.x;
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += step) {
    int64_t rest = i, so = 0, dof = 0;
    for (int d = rank - 1; d > 0; --d) {
      const int64_t q = rest / sh.extent[d], r = rest - q * sh.extent[d];
      so += r * sh.src_stride[d];
      dof += r * sh.dst_stride[d];
      rest = q;
    }
    so += rest * sh.src_stride[0];
    dof += rest * sh.dst_stride[0];
    *reinterpret_cast<U*>(dst + dof) = *reinterpret_cast<const U*>(src + so);
  }
}
// (src, dst, total units, rank >= 1, shape) ; every address formed is aligned to the unit.
#define MTRT_COPY_STRIDED(BYTES, U)                                                                                   \
  extern "C" __global__ void __launch_bounds__(256) mtrt_copy_strided_b##BYTES(                                       \
      const uint8_t* src, uint8_t* dst, int64_t total, int32_t rank, StridedCopyShape shape) {                        \
    copy_strided<U>(src, dst, total, rank, shape); }
MTRT_COPY_STRIDED(1, uint8_t)
MTRT_COPY_STRIDED(2, uint16_t)
MTRT_COPY_STRIDED(4, uint32_t)
MTRT_COPY_STRIDED(8, u32x2)
MTRT_COPY_STRIDED(16, u32x4)
