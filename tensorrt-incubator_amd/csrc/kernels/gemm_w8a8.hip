// W8A8 GEMM cluster for gfx950:
//     acc[m,n] = sum_k i32(a[m,k]) * i32(w[k,n])                 (exact int32)
//     y[m,n]   = f16((f32(acc[m,n]) * a_scale[m]) * w_scale[n])   (two f32 roundings, then f16)
// i.e. the dot_general + per-token / per-output-channel dequantize epilogue of a
// quantized Linear (tripy/nvtripy/frontend/module/linear.py:112-151), which the
// reference realises as a plain FMA loop nest without matrix cores
// (mlir-tensorrt/kernel/test/Kernel/TransformSchedules/fallback-schedule-matmul.mlir:24).
//
// Matrix cores want both operands contiguous along K per row/column.  Activations
// [M,K] already are.  Weights arrive as [K,N] (N contiguous); they are constants of
// the program, so they are re-laid once into [N,K] by mtrt_w8_prepack_kn_to_nk and
// the GEMM consumes that.  The main loop (tiling, pipeline, LDS layout, tile order,
// epilogue staging) is the shared one in gemm_core.hpp with v_mfma_i32_32x32x32_i8.
#include "gemm_core.hpp"

namespace gemm_w8a8_cluster {

using namespace mtrt_dev;
using gemm_core::v4i;
typedef int v16i __attribute__((ext_vector_type(16)));

struct I8Traits {
  using Acc = v16i;
  static __device__ __forceinline__ Acc zero() {
    Acc z;
#pragma unroll
    for (int r = 0; r < 16; ++r) z[r] = 0;
    return z;
  }
  static __device__ __forceinline__ Acc mfma(v4i a, v4i b, Acc c) { return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0); }
};

struct ScaleEpilogue {
  const float* a_scale;
  const float* w_scale;
  const float* sa;                                   // a_scale of this tile's 256 rows, in LDS
  const float* sw;                                   // w_scale of this tile's 256 columns, in LDS
  float as;
  __device__ __forceinline__ void setup(int8_t* scratch, int64_t m0, int64_t M, int64_t n0, int64_t N) {
    float* dst = reinterpret_cast<float*>(scratch);
    const int64_t row = m0 + threadIdx.x, col = n0 + threadIdx.x;   // 256 threads: 256 rows, 256 columns
    dst[threadIdx.x] = row < M ? a_scale[row] : 0.0f;
    dst[256 + threadIdx.x] = col < N ? w_scale[col] : 0.0f;
    sa = dst;
    sw = dst + 256;
  }
  __device__ __forceinline__ void row(int row_in_tile) { as = sa[row_in_tile]; }
  __device__ __forceinline__ void convert4(const v16i& acc, int q, int col_in_tile, uint32_t (&bits)[4]) const {
    const f32x4 ws = *reinterpret_cast<const f32x4*>(sw + col_in_tile);
#pragma unroll
    for (int e = 0; e < 4; ++e) bits[e] = f32_to_f16_bits((float(acc[4 * q + e]) * as) * ws[e]);
  }
};

// The entry points below have C linkage; they sit inside the namespace only so that
// its helper names do not meet those of the other clusters in the one-module build.

// (a [M,K] i8, w_nk [N,K] i8, a_scale [M] f32, w_scale [N] f32, y [M,N] f16, M, K, N, full_panels) ; K % 128 == 0,
// a and w_nk 16-byte aligned, both below 4 GiB.  The first full_panels * 256 columns are computed in
// 256 x 256 tiles, the rest in 256 x 128 tiles: with one workgroup per compute unit a launch runs in
// rounds, and a last round that would use few of the units is cut into twice as many tiles of half
// the length.  grid = padded_blocks(full_panels, tiles_m) + padded_blocks(half panels, tiles_m), block = 256.
extern "C" __global__ void __launch_bounds__(gemm_core::THREADS, 1) mtrt_gemm_w8a8_nk(
    const int8_t* __restrict__ a, const int8_t* __restrict__ w, const float* __restrict__ a_scale,
    const float* __restrict__ w_scale, uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N, int64_t full_panels) {
  __shared__ __attribute__((aligned(16))) int8_t lds[gemm_core::LDS_BYTES];
  const int64_t tiles_m = (M + gemm_core::BM - 1) / gemm_core::BM;
  const int64_t full_blocks = gemm_core::padded_blocks(full_panels, tiles_m);
  ScaleEpilogue epi{a_scale, w_scale, nullptr, nullptr, 0.0f};
  int64_t tile_m, panel;
  if (int64_t(blockIdx.x) < full_blocks) {
    if (!gemm_core::tile_of(blockIdx.x, tiles_m, full_panels, tile_m, panel)) return;
    gemm_core::run<I8Traits, 4>(a, w, K, epi, y, M, N, K / gemm_core::BKB, tile_m * 256, panel * 256, lds);
  } else {
    const int64_t n_full = full_panels * 256;
    if (!gemm_core::tile_of(blockIdx.x - full_blocks, tiles_m, (N - n_full + 127) / 128, tile_m, panel)) return;
    gemm_core::run<I8Traits, 2>(a, w, K, epi, y, M, N, K / gemm_core::BKB, tile_m * 256, n_full + panel * 128, lds);
  }
}

// Any K (no alignment needs): one output element per lane, plain loops.  Serves
// shapes the MFMA kernel does not take; not a fast path.
extern "C" __global__ void __launch_bounds__(256) mtrt_gemm_w8a8_nk_any(
    const int8_t* __restrict__ a, const int8_t* __restrict__ w, const float* __restrict__ a_scale,
    const float* __restrict__ w_scale, uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N) {
  const int64_t total = M * N;
  for (int64_t e = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; e < total; e += int64_t(gridDim.x) * blockDim.x) {
    const int64_t m = e / N, n = e - m * N;
    int acc = 0;
    for (int64_t k = 0; k < K; ++k) acc += int(a[m * K + k]) * int(w[n * K + k]);
    y[e] = uint16_t(f32_to_f16_bits((float(acc) * a_scale[m]) * w_scale[n]));
  }
}

// Weight re-layout [K,N] -> [N,K], bytes.  64 x 64 tiles through LDS; both the global
// read and the global write are contiguous.  (w_kn, w_nk, K, N) grid = ceil(K/64)*ceil(N/64).
extern "C" __global__ void __launch_bounds__(256) mtrt_w8_prepack_kn_to_nk(const int8_t* __restrict__ w_kn,
                                                                         int8_t* __restrict__ w_nk, int64_t K, int64_t N) {
  __shared__ int8_t tile[64][65];
  const int64_t tiles_n = (N + 63) / 64;
  const int64_t k0 = int64_t(blockIdx.x / tiles_n) * 64, n0 = int64_t(blockIdx.x % tiles_n) * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int64_t k = k0 + ty + 4 * i, n = n0 + tx;
    if (k < K && n < N) tile[ty + 4 * i][tx] = w_kn[k * N + n];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int64_t n = n0 + ty + 4 * i, k = k0 + tx;
    if (k < K && n < N) w_nk[n * K + k] = tile[tx][ty + 4 * i];
  }
}

}  // namespace gemm_w8a8_cluster
