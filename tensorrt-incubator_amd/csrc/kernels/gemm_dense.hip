// Dense Linear: y[m,n] = narrow(sum_k f32(x[m,k]) * f32(w[n,k]) (+ f32(bias[n]))), f32 accumulation, all
// operands of one float type.  This is the float matmul of the quantized Linear in its fake-quant form
//   tripy/nvtripy/frontend/module/linear.py:112-151   (out = x' @ W'^T + b on the dequantized operands)
// for the parameter combinations the integer / int4 matrix-core clusters cannot express (f8 codes, scales
// along the input features, int4 blocks along the output features) and for the unquantized module.  The
// reference's own generator emits an FMA loop nest for such a matmul
// (mlir-tensorrt/kernel/test/Kernel/TransformSchedules/fallback-schedule-matmul.mlir:24); this is the same
// class of kernel, tiled through LDS: 64 x 64 outputs per workgroup, 4 x 4 per lane, K in slices of 16.
// w is [N,K] (K contiguous), the module's own weight layout; any M, N, K; no alignment needs.
#include "common.hpp"

using namespace mtrt_dev;

namespace dense_cluster {

constexpr int kDenseTile = 64, kDenseK = 16;

template <typename X>
__device__ __forceinline__ void dense_body(const typename X::storage* __restrict__ x, const typename X::storage* __restrict__ w,
                                           const typename X::storage* __restrict__ bias, typename X::storage* __restrict__ y,
                                           int64_t M, int64_t K, int64_t N) {
  __shared__ float xs[kDenseK][kDenseTile + 1];
  __shared__ float ws[kDenseK][kDenseTile + 1];
  const int64_t tiles_n = (N + kDenseTile - 1) / kDenseTile;
  const int64_t m0 = int64_t(blockIdx.x / tiles_n) * kDenseTile, n0 = int64_t(blockIdx.x % tiles_n) * kDenseTile;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;       // lane's 4 x 4 block: rows 4*ty.., columns 4*tx..
  const int lk = threadIdx.x & 15, lr = threadIdx.x >> 4;       // loader: k index, row index (+16 per step)
  float acc[4][4] = {};
  for (int64_t k0 = 0; k0 < K; k0 += kDenseK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = lr + 16 * i;
      const int64_t k = k0 + lk;
      xs[lk][r] = (m0 + r < M && k < K) ? Tile<X>::load1(x + (m0 + r) * K + k) : 0.0f;
      ws[lk][r] = (n0 + r < N && k < K) ? Tile<X>::load1(w + (n0 + r) * K + k) : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kDenseK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { a[i] = xs[kk][4 * ty + i]; b[i] = ws[kk][4 * tx + i]; }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t m = m0 + 4 * ty + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t n = n0 + 4 * tx + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (bias) v = v + Tile<X>::load1(bias + n);
      Tile<X>::store1(y + m * N + n, v);
    }
  }
}

}  // namespace dense_cluster

// (x [M,K], w [N,K], bias [N] or null, y [M,N], M, K, N) ; grid = ceil(M/64) * ceil(N/64), block = 256
#define MTRT_DENSE_KERNEL(XN, XT)                                                                                  \
  extern "C" __global__ void __launch_bounds__(256) mtrt_gemm_dense_##XN(                                          \
      const XT::storage* x, const XT::storage* w, const XT::storage* bias, XT::storage* y, int64_t M, int64_t K,   \
      int64_t N) { dense_cluster::dense_body<XT>(x, w, bias, y, M, K, N); }
MTRT_DENSE_KERNEL(f32, F32)
MTRT_DENSE_KERNEL(f16, F16)
MTRT_DENSE_KERNEL(bf16, BF16)
