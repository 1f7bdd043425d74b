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
