// Dense Linear: y[m,n] = narrow(sum_k f32(x[m,k]) * f32(w[n,k]) (+ f32(bias[n]))), f32 accumulation, all
// operands of one float type.  This is the float matmul of the quantized Linear in its fake-quant form
//   tripy/nvtripy/frontend/module/linear.py:112-151   (out = x' @ W'^T + b on the dequantized operands)
// for the parameter combinations the integer / int4 matrix-core clusters cannot express (f8 codes, scales
// along the input features, int4 blocks along the output features) and for the unquantized module.  The
// reference's own generator emits an FMA loop nest for such a matmul
// (mlir-tensorrt/kernel/test/Kernel/TransformSchedules/fallback-schedule-matmul.mlir:24); this is the same
// class of kernel, tiled through LDS: 64 x 64 outputs per workgroup, 4 x 4 per lane, K in slices of 16.
// w is [N,K] (K contiguous), the module's own weight layout; any M, N, K; no alignment needs.  It only serves
// K = 0 now: every other shape runs on the matrix cores (mtrt_gemm_dense_edge_* for rows that are not whole slices).
// 16-bit operands whose rows are whole 128-byte slices (K % 64 == 0, 16-byte aligned) go to the matrix cores
// instead (mtrt_gemm_dense_mfma_*): both operands are K-contiguous per row, which is the form the shared tile
// loop of gemm_core.hpp takes (both panels through LDS, 256 x 256 tiles, v_mfma_f32_32x32x16_{f16,bf16}; a
// product of two 16-bit floats is exact in f32), with the bias added to the f32 sum before the one narrowing.
#include "gemm_core.hpp"

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

// ---- matrix-core form for f16 / bf16 --------------------------------------------------------------------
using gemm_core::v4i;
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8b __attribute__((ext_vector_type(8)));

template <typename X> struct HalfTraits;
template <> struct HalfTraits<F16> {
  using Acc = v16f;
  using Scalar = float;
  static __device__ __forceinline__ Acc zero() {
    Acc z;
#pragma unroll
    for (int r = 0; r < 16; ++r) z[r] = 0.0f;
    return z;
  }
  static __device__ __forceinline__ Acc mfma(v4i a, v4i b, Acc c) {
    union { v4i i; v8h h; } ua, ub;
    ua.i = a; ub.i = b;
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(ua.h, ub.h, c, 0, 0, 0);
  }
};
template <> struct HalfTraits<BF16> {
  using Acc = v16f;
  using Scalar = float;
  static __device__ __forceinline__ Acc zero() { return HalfTraits<F16>::zero(); }
  static __device__ __forceinline__ Acc mfma(v4i a, v4i b, Acc c) {
    union { v4i i; v8b h; } ua, ub;
    ua.i = a; ub.i = b;
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(ua.h, ub.h, c, 0, 0, 0);
  }
};

// f32 operands: a 16-byte fragment holds four k values per lane, and v_mfma_f32_32x32x2_f32 takes one per lane (the two
// halves of the wave supplying its two k values), so a fragment pair is four chained instructions; which k values
// meet in one instruction does not matter as long as both operands agree.
struct F32Traits {
  using Acc = v16f;
  using Scalar = float;
  static __device__ __forceinline__ Acc zero() { return HalfTraits<F16>::zero(); }
  static __device__ __forceinline__ Acc mfma(v4i a, v4i b, Acc c) {
#pragma unroll
    for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_32x32x2f32(bits_to_f32(uint32_t(a[e])), bits_to_f32(uint32_t(b[e])), c, 0, 0, 0);
    return c;
  }
};
struct BiasF32Epilogue {
  const float* bias;
  __device__ __forceinline__ void finish4(float (&v)[4], int64_t col, int64_t N) const {
    if (!bias) return;
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (col + e < N) v[e] = v[e] + bias[col + e];
  }
};

template <typename X> __device__ __forceinline__ uint32_t narrow16(float v);
template <> __device__ __forceinline__ uint32_t narrow16<F16>(float v) { return f32_to_f16_bits(v); }
template <> __device__ __forceinline__ uint32_t narrow16<BF16>(float v) { return f32_to_bf16_bits(v); }
template <typename X> __device__ __forceinline__ uint32_t narrow16x2(float lo, float hi);
template <> __device__ __forceinline__ uint32_t narrow16x2<F16>(float lo, float hi) { return f32x2_to_f16x2_bits(lo, hi); }
template <> __device__ __forceinline__ uint32_t narrow16x2<BF16>(float lo, float hi) { return f32x2_to_bf16x2_bits(lo, hi); }

// y = narrow(acc + f32(bias[n])) (no addition without a bias, as in the kernel above)
template <typename X>
struct BiasEpilogue {
  const typename X::storage* bias;
  const float* sb;                                   // bias of this tile's 256 columns as f32, in LDS
  f32x4 br[2][4];
  __device__ __forceinline__ void setup(int8_t* scratch, int64_t, int64_t, int64_t n0, int64_t N) {
    float* dst = reinterpret_cast<float*>(scratch);
    const int64_t col = n0 + threadIdx.x;             // 256 threads: 256 columns
    if (threadIdx.x < 256) dst[threadIdx.x] = (bias && col < N) ? Tile<X>::load1(bias + col) : 0.0f;
    sb = dst;
  }
  __device__ __forceinline__ void row(int) {}
  template <int HC>
  __device__ __forceinline__ void columns(int first_col_in_tile) {
#pragma unroll
    for (int jj = 0; jj < HC; ++jj)
#pragma unroll
      for (int q = 0; q < 4; ++q) br[jj][q] = *reinterpret_cast<const f32x4*>(sb + first_col_in_tile + jj * 32 + q * 8);
  }
  __device__ __forceinline__ void convert4(const v16f& acc, int q, int jj, uint32_t (&words)[2]) const {
#pragma unroll
    for (int e = 0; e < 4; e += 2) {
      float v0 = acc[4 * q + e], v1 = acc[4 * q + e + 1];
      if (bias) {
        v0 = v0 + br[jj][q][e];
        v1 = v1 + br[jj][q][e + 1];
      }
      words[e >> 1] = narrow16x2<X>(v0, v1);
    }
  }
};

template <typename X>
__device__ __forceinline__ void dense_mfma_body(const typename X::storage* __restrict__ x, const typename X::storage* __restrict__ w,
                                                const typename X::storage* __restrict__ bias, uint16_t* __restrict__ y, int64_t M,
                                                int64_t K, int64_t N, int64_t full_panels, int8_t* lds) {
  const int64_t tiles_m = (M + gemm_core::BM - 1) / gemm_core::BM;
  const int64_t full_blocks = gemm_core::even_blocks(full_panels * tiles_m);
  BiasEpilogue<X> epi{bias, nullptr, {}};
  const int8_t* a8 = reinterpret_cast<const int8_t*>(x);
  const int8_t* w8 = reinterpret_cast<const int8_t*>(w);
  int64_t tile_m, panel;
  if (int64_t(blockIdx.x) < full_blocks) {
    if (!gemm_core::tile_of_even(blockIdx.x, uint32_t(full_blocks), tiles_m, full_panels, tiles_m, tile_m, panel)) return;
    gemm_core::run<HalfTraits<X>, 4>(a8, w8, K * 2, epi, y, M, N, K * 2 / gemm_core::BKB, tile_m * 256, panel * 256, lds);
  } else {
    const int64_t n_full = full_panels * 256;
    if (!gemm_core::tile_of_even(blockIdx.x - uint32_t(full_blocks), gridDim.x - uint32_t(full_blocks), tiles_m, (N - n_full + 127) / 128,
                                 tiles_m, tile_m, panel))
      return;
    gemm_core::run<HalfTraits<X>, 2>(a8, w8, K * 2, epi, y, M, N, K * 2 / gemm_core::BKB, tile_m * 256, n_full + panel * 128, lds);
  }
}

__device__ __forceinline__ void dense_mfma_f32_body(const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ bias,
                                                    float* __restrict__ y, int64_t M, int64_t K, int64_t N, int64_t full_panels,
                                                    int8_t* lds) {
  const int64_t tiles_m = (M + gemm_core::BM - 1) / gemm_core::BM;
  const int64_t full_blocks = gemm_core::even_blocks(full_panels * tiles_m);
  BiasF32Epilogue epi{bias};
  const int8_t* a8 = reinterpret_cast<const int8_t*>(x);
  const int8_t* w8 = reinterpret_cast<const int8_t*>(w);
  int64_t tile_m, panel;
  if (int64_t(blockIdx.x) < full_blocks) {
    if (!gemm_core::tile_of_even(blockIdx.x, uint32_t(full_blocks), tiles_m, full_panels, tiles_m, tile_m, panel)) return;
    gemm_core::run<F32Traits, 4>(a8, w8, K * 4, epi, y, M, N, K * 4 / gemm_core::BKB, tile_m * 256, panel * 256, lds);
  } else {
    const int64_t n_full = full_panels * 256;
    if (!gemm_core::tile_of_even(blockIdx.x - uint32_t(full_blocks), gridDim.x - uint32_t(full_blocks), tiles_m, (N - n_full + 127) / 128,
                                 tiles_m, tile_m, panel))
      return;
    gemm_core::run<F32Traits, 2>(a8, w8, K * 4, epi, y, M, N, K * 4 / gemm_core::BKB, tile_m * 256, n_full + panel * 128, lds);
  }
}

// Epilogues of the any-shape tile loop (gemm_core::edge): the same sum + bias, one narrowing.
template <typename X>
struct EdgeBiasEpilogue {
  const typename X::storage* bias;
  __device__ __forceinline__ void row(int64_t, bool) {}
  __device__ __forceinline__ uint32_t finish(float acc, int64_t col, bool valid) const {
    if (bias && valid) acc = acc + Tile<X>::load1(bias + col);
    return narrow16<X>(acc);
  }
};
struct EdgeBiasF32Epilogue {
  const float* bias;
  __device__ __forceinline__ void row(int64_t, bool) {}
  __device__ __forceinline__ float finish(float acc, int64_t col, bool valid) const { return bias && valid ? acc + bias[col] : acc; }
};

// Epilogues of the up-to-32-rows kernel (gemm_core::rows32)
template <typename X>
struct RowsBiasEpilogue {
  const typename X::storage* bias;
  __device__ __forceinline__ uint32_t finish(float sum, int64_t, int64_t col) const {
    if (bias) sum = sum + Tile<X>::load1(bias + col);
    return narrow16<X>(sum);
  }
};
struct RowsBiasF32Epilogue {
  const float* bias;
  __device__ __forceinline__ float finish(float sum, int64_t, int64_t col) const { return bias ? sum + bias[col] : sum; }
};

}  // namespace dense_cluster

// f32 operands: (x [M,K], w [N,K], bias [N] or null, y [M,N], M, K, N, full_panels) ; K % 32 == 0, x and w 16-byte aligned
// and below 4 GiB each; tiles, grid and block as for the 16-bit kernels below.
extern "C" __global__ void __launch_bounds__(gemm_core::THREADS, 1) mtrt_gemm_dense_mfma_f32(
    const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ bias, float* __restrict__ y, int64_t M,
    int64_t K, int64_t N, int64_t full_panels) {
  __shared__ __attribute__((aligned(16))) int8_t lds[gemm_core::LDS_BYTES];
  dense_cluster::dense_mfma_f32_body(x, w, bias, y, M, K, N, full_panels, lds);
}

// (x [M,K], w [N,K], bias [N] or null, y [M,N], M, K, N, full_panels) ; K % 64 == 0, x and w 16-byte aligned and below
// 4 GiB each; tiles and grid as mtrt_gemm_w8a8_nk (256 x 256 for the first full_panels * 256 columns, 256 x 128 after),
// block = 256.
#define MTRT_DENSE_MFMA_KERNEL(XN, XT)                                                                             \
  extern "C" __global__ void __launch_bounds__(gemm_core::THREADS, 1) mtrt_gemm_dense_mfma_##XN(                   \
      const XT::storage* __restrict__ x, const XT::storage* __restrict__ w, const XT::storage* __restrict__ bias,  \
      uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N, int64_t full_panels) {                            \
    __shared__ __attribute__((aligned(16))) int8_t lds[gemm_core::LDS_BYTES];                                      \
    dense_cluster::dense_mfma_body<XT>(x, w, bias, y, M, K, N, full_panels, lds);                                  \
  }
MTRT_DENSE_MFMA_KERNEL(f16, F16)
MTRT_DENSE_MFMA_KERNEL(bf16, BF16)

// Up to 32 rows, weights read once as whole rows (gemm_core::rows32): (x [M,K], w [N,K], bias or null, y, M <= 32, K, N) ;
// rows in whole 128-byte slices, x and w 16-byte aligned; grid: any, block = 512.
extern "C" __global__ void __launch_bounds__(512) mtrt_gemm_dense_rows32_f32(
    const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ bias, float* __restrict__ y, int64_t M,
    int64_t K, int64_t N) {
  __shared__ __attribute__((aligned(16))) int8_t lds[gemm_core::rows32::lds_bytes<8>()];
  dense_cluster::RowsBiasF32Epilogue epi{bias};
  gemm_core::rows32::run<dense_cluster::F32Traits, 8>(reinterpret_cast<const int8_t*>(x), reinterpret_cast<const int8_t*>(w), K * 4, epi, y, M, N, lds);
}
#define MTRT_DENSE_ROWS32_KERNEL(XN, XT)                                                                           \
  extern "C" __global__ void __launch_bounds__(512) mtrt_gemm_dense_rows32_##XN(                                   \
      const XT::storage* __restrict__ x, const XT::storage* __restrict__ w, const XT::storage* __restrict__ bias,  \
      uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N) {                                                 \
    __shared__ __attribute__((aligned(16))) int8_t lds[gemm_core::rows32::lds_bytes<8>()];                         \
    dense_cluster::RowsBiasEpilogue<XT> epi{bias};                                                                 \
    gemm_core::rows32::run<dense_cluster::HalfTraits<XT>, 8>(reinterpret_cast<const int8_t*>(x), reinterpret_cast<const int8_t*>(w), K * 2, \
                                                             epi, y, M, N, lds);                                   \
  }
MTRT_DENSE_ROWS32_KERNEL(f16, F16)
MTRT_DENSE_ROWS32_KERNEL(bf16, BF16)
// ... and up to 64 rows: two activation row tiles against each weight fragment
extern "C" __global__ void __launch_bounds__(512) mtrt_gemm_dense_rows64_f32(
    const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ bias, float* __restrict__ y, int64_t M,
    int64_t K, int64_t N) {
  __shared__ __attribute__((aligned(16))) int8_t lds[gemm_core::rows32::lds_bytes<8, 2>()];
  dense_cluster::RowsBiasF32Epilogue epi{bias};
  gemm_core::rows32::run<dense_cluster::F32Traits, 8, 2>(reinterpret_cast<const int8_t*>(x), reinterpret_cast<const int8_t*>(w), K * 4, epi, y, M, N, lds);
}
#define MTRT_DENSE_ROWS64_KERNEL(XN, XT)                                                                           \
  extern "C" __global__ void __launch_bounds__(512) mtrt_gemm_dense_rows64_##XN(                                   \
      const XT::storage* __restrict__ x, const XT::storage* __restrict__ w, const XT::storage* __restrict__ bias,  \
      uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N) {                                                 \
    __shared__ __attribute__((aligned(16))) int8_t lds[gemm_core::rows32::lds_bytes<8, 2>()];                      \
    dense_cluster::RowsBiasEpilogue<XT> epi{bias};                                                                 \
    gemm_core::rows32::run<dense_cluster::HalfTraits<XT>, 8, 2>(reinterpret_cast<const int8_t*>(x), reinterpret_cast<const int8_t*>(w),     \
                                                                K * 2, epi, y, M, N, lds);                         \
  }
MTRT_DENSE_ROWS64_KERNEL(f16, F16)
MTRT_DENSE_ROWS64_KERNEL(bf16, BF16)
// ... and up to 128 rows: four row tiles, four waves (block = 256)
extern "C" __global__ void __launch_bounds__(256) mtrt_gemm_dense_rows128_f32(
    const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ bias, float* __restrict__ y, int64_t M,
    int64_t K, int64_t N) {
  __shared__ __attribute__((aligned(16))) int8_t lds[gemm_core::rows32::lds_bytes<4, 4>()];
  dense_cluster::RowsBiasF32Epilogue epi{bias};
  gemm_core::rows32::run<dense_cluster::F32Traits, 4, 4>(reinterpret_cast<const int8_t*>(x), reinterpret_cast<const int8_t*>(w), K * 4, epi, y, M, N, lds);
}
#define MTRT_DENSE_ROWS128_KERNEL(XN, XT)                                                                          \
  extern "C" __global__ void __launch_bounds__(256) mtrt_gemm_dense_rows128_##XN(                                  \
      const XT::storage* __restrict__ x, const XT::storage* __restrict__ w, const XT::storage* __restrict__ bias,  \
      uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N) {                                                 \
    __shared__ __attribute__((aligned(16))) int8_t lds[gemm_core::rows32::lds_bytes<4, 4>()];                      \
    dense_cluster::RowsBiasEpilogue<XT> epi{bias};                                                                 \
    gemm_core::rows32::run<dense_cluster::HalfTraits<XT>, 4, 4>(reinterpret_cast<const int8_t*>(x), reinterpret_cast<const int8_t*>(w),     \
                                                                K * 2, epi, y, M, N, lds);                         \
  }
MTRT_DENSE_ROWS128_KERNEL(f16, F16)
MTRT_DENSE_ROWS128_KERNEL(bf16, BF16)

// Any K and any alignment on the matrix cores: (x [M,K], w [N,K], bias [N] or null, y [M,N], M, K, N) ; grid: any
// (128 x 128 tiles dealt round-robin), block = 256.
extern "C" __global__ void __launch_bounds__(256) mtrt_gemm_dense_edge_f32(
    const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ bias, float* __restrict__ y, int64_t M,
    int64_t K, int64_t N) {
  __shared__ __attribute__((aligned(16))) int8_t lds[gemm_core::edge::kLdsBytes];
  dense_cluster::EdgeBiasF32Epilogue epi{bias};
  gemm_core::edge::run<dense_cluster::F32Traits>(reinterpret_cast<const int8_t*>(x), reinterpret_cast<const int8_t*>(w), K * 4, epi, y, M, N, lds);
}
#define MTRT_DENSE_EDGE_KERNEL(XN, XT)                                                                             \
  extern "C" __global__ void __launch_bounds__(256) mtrt_gemm_dense_edge_##XN(                                     \
      const XT::storage* __restrict__ x, const XT::storage* __restrict__ w, const XT::storage* __restrict__ bias,  \
      uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N) {                                                 \
    __shared__ __attribute__((aligned(16))) int8_t lds[gemm_core::edge::kLdsBytes];                                \
    dense_cluster::EdgeBiasEpilogue<XT> epi{bias};                                                                 \
    gemm_core::edge::run<dense_cluster::HalfTraits<XT>>(reinterpret_cast<const int8_t*>(x), reinterpret_cast<const int8_t*>(w), K * 2, epi, y, \
                                                        M, N, lds);                                                \
  }
MTRT_DENSE_EDGE_KERNEL(f16, F16)
MTRT_DENSE_EDGE_KERNEL(bf16, BF16)

// (x [M,K], w [N,K], bias [N] or null, y [M,N], M, K, N) ; grid = ceil(M/64) * ceil(N/64), block = 256
#define MTRT_DENSE_KERNEL(XN, XT)                                                                                  \
  extern "C" __global__ void __launch_bounds__(256) mtrt_gemm_dense_##XN(                                          \
      const XT::storage* x, const XT::storage* w, const XT::storage* bias, XT::storage* y, int64_t M, int64_t K,   \
      int64_t N) { dense_cluster::dense_body<XT>(x, w, bias, y, M, K, N); }
MTRT_DENSE_KERNEL(f32, F32)
MTRT_DENSE_KERNEL(f16, F16)
MTRT_DENSE_KERNEL(bf16, BF16)
