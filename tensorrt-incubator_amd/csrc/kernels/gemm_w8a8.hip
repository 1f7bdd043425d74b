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
// the GEMM consumes that.
//
// GEMM kernel: one workgroup of 4 waves computes a 256 x 128 tile of y.  Per 128-byte
// K slice the A (256 x 128 B) and W (128 x 128 B) panels go global -> registers ->
// LDS (double buffered; the loads of slice t+1 are in flight while slice t is being
// multiplied), each wave then owns a 128 x 64 sub-tile = 4 x 2 MFMA tiles of
// v_mfma_i32_32x32x32_i8, 128 accumulator registers per lane.  LDS rows are 128 B
// (8 chunks of 16 B); chunk c of row r lives at chunk position c ^ ((r >> 1) & 7), which
// spreads the 16-byte fragment reads of 32 consecutive rows over all banks.
// The epilogue applies both scales in the order above and stores f16.
#include "common.hpp"

using namespace mtrt_dev;

namespace gemm_w8a8_cluster {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int BM = 256, BN = 128, BK = 128;          // BK in bytes (= int8 elements)
constexpr int THREADS = 256;
constexpr int A_CHUNKS = BM * BK / 16 / THREADS;     // 16-byte loads per thread per slice: 8
constexpr int B_CHUNKS = BN * BK / 16 / THREADS;     // 4
constexpr int A_BYTES = BM * BK, B_BYTES = BN * BK;

__device__ __forceinline__ int lds_off(int row, int chunk) { return row * BK + ((chunk ^ ((row >> 1) & 7)) << 4); }

struct Staging {
  v4i a[A_CHUNKS];
  v4i b[B_CHUNKS];
};

__device__ __forceinline__ void load_slice(Staging& st, const int8_t* __restrict__ a, const int8_t* __restrict__ w,
                                           int64_t M, int64_t N, int64_t K, int64_t m0, int64_t n0, int64_t k0) {
  const int t = threadIdx.x;
  const int ch = t & 7;
#pragma unroll
  for (int i = 0; i < A_CHUNKS; ++i) {
    int64_t row = m0 + (t >> 3) + 32 * i;
    row = row < M ? row : M - 1;                     // rows past the edge re-read the last row; never stored
    st.a[i] = *reinterpret_cast<const v4i*>(a + row * K + k0 + ch * 16);
  }
#pragma unroll
  for (int i = 0; i < B_CHUNKS; ++i) {
    int64_t row = n0 + (t >> 3) + 32 * i;
    row = row < N ? row : N - 1;
    st.b[i] = *reinterpret_cast<const v4i*>(w + row * K + k0 + ch * 16);
  }
}

__device__ __forceinline__ void store_slice(const Staging& st, int8_t* lds_a, int8_t* lds_b) {
  const int t = threadIdx.x;
  const int ch = t & 7;
#pragma unroll
  for (int i = 0; i < A_CHUNKS; ++i) *reinterpret_cast<v4i*>(lds_a + lds_off((t >> 3) + 32 * i, ch)) = st.a[i];
#pragma unroll
  for (int i = 0; i < B_CHUNKS; ++i) *reinterpret_cast<v4i*>(lds_b + lds_off((t >> 3) + 32 * i, ch)) = st.b[i];
}

// The entry points below have C linkage; they sit inside the namespace only so that
// its helper names do not meet those of the other clusters in the one-module build.

// (a [M,K] i8, w_nk [N,K] i8, a_scale [M] f32, w_scale [N] f32, y [M,N] f16, M, K, N) ; K % 128 == 0,
// a and w_nk 16-byte aligned.  grid = ceil(M/256) * ceil(N/128), block = 256.
extern "C" __global__ void __launch_bounds__(THREADS) mtrt_gemm_w8a8_nk(
    const int8_t* __restrict__ a, const int8_t* __restrict__ w, const float* __restrict__ a_scale,
    const float* __restrict__ w_scale, uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N) {
  __shared__ __attribute__((aligned(16))) int8_t lds[2 * (A_BYTES + B_BYTES)];
  constexpr int kStage = A_BYTES + B_BYTES;         // stage s: A panel at s*kStage, W panel right after it

  // Tile order: consecutive workgroups walk down M inside one N panel, so the
  // workgroups in flight at any time share a few W panels and all of A.
  const int64_t tiles_m = (M + BM - 1) / BM;
  const int64_t m0 = int64_t(blockIdx.x % tiles_m) * BM;
  const int64_t n0 = int64_t(blockIdx.x / tiles_m) * BN;

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;           // 2 x 2 waves: 128 x 64 each
  const int frow = lane & 31, fhalf = lane >> 5;

  v16i acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  Staging st;
  load_slice(st, a, w, M, N, K, m0, n0, 0);
  store_slice(st, lds, lds + A_BYTES);
  __syncthreads();

  const int64_t slices = K / BK;
  for (int64_t s = 0; s < slices; ++s) {
    const int cur = int(s & 1);
    const int8_t* pa = lds + cur * kStage;
    const int8_t* pb = pa + A_BYTES;
    if (s + 1 < slices) load_slice(st, a, w, M, N, K, m0, n0, (s + 1) * BK);
#pragma unroll
    for (int ks = 0; ks < BK / 32; ++ks) {
      v4i fa[4], fb[2];
      const int chunk = ks * 2 + fhalf;
#pragma unroll
      for (int i = 0; i < 4; ++i) fa[i] = *reinterpret_cast<const v4i*>(pa + lds_off(wm * 128 + i * 32 + frow, chunk));
#pragma unroll
      for (int j = 0; j < 2; ++j) fb[j] = *reinterpret_cast<const v4i*>(pb + lds_off(wn * 64 + j * 32 + frow, chunk));
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    if (s + 1 < slices) store_slice(st, lds + (cur ^ 1) * kStage, lds + (cur ^ 1) * kStage + A_BYTES);
    __syncthreads();
  }

  // Epilogue.  In a 32x32 accumulator tile lane l holds column (l & 31) and rows
  // 8*(r/4) + 4*(l >> 5) + (r % 4), r = 0..15.
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int64_t col = n0 + wn * 64 + j * 32 + frow;
    if (col >= N) continue;
    const float ws = w_scale[col];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t row = m0 + wm * 128 + i * 32 + (r >> 2) * 8 + fhalf * 4 + (r & 3);
        if (row < M) y[row * N + col] = uint16_t(f32_to_f16_bits((float(acc[i][j][r]) * a_scale[row]) * ws));
      }
    }
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
