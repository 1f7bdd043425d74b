// amax per scale element: the reduction that produces the scales of the per-channel and block-wise modes of
// tensorrt.quantize (TensorRTOps.td:3133-3194), as the calibration flow computes them
//   scale = amax.float() / maxbound        tripy/examples/nanogpt/weight_loader.py:67-68
//   int4 blocks: amax reshaped per block   weight_loader.py:102-115
// The tensor is viewed as row-major [d0, d1] and the scale addressing is the one of qdq.hip:
//   row : scale[row % nb]            one scale per row (nb = d0: per-token / per-output-channel, blocks along the last
//                                    axis) or per channel of a middle axis (rows r, r + nb, ... share a scale)
//   col : scale[(row / nb) * d1 + c] blocks of nb rows per column (nb = d0: per-channel on the last axis)
// For every scale element: amax = max |f32(x)| over the elements that address it (exact in any order, so the result
// is bit-identical to a sequential host reduction), scale = amax / qmax (one IEEE divide).  The reference's generated
// reduction walks each row serially per thread (mlir-tensorrt/kernel/lib/Utils/TilingUtils.cpp:669-677); here a wave
// owns a scale (row kinds) or a workgroup a 64-vector-wide strip of one block (col kind), 128-bit loads throughout.
#include "common.hpp"

namespace amax_scales_cluster {

using namespace mtrt_dev;
using namespace amax_cluster;

// max |.| of each of the G elements of a vector, as orderable bit patterns (see AbsBits)
template <typename X> struct AbsEach;
template <> struct AbsEach<F32> {
  static constexpr int G = 4;
  static __device__ __forceinline__ void acc(u32x4 t, uint32_t (&m)[4]) {
#pragma unroll
    for (int k = 0; k < 4; ++k) { const uint32_t a = t[k] & 0x7FFFFFFFu; m[k] = m[k] > a ? m[k] : a; }
  }
};
template <> struct AbsEach<BF16> {
  static constexpr int G = 8;
  static __device__ __forceinline__ void acc(u32x4 t, uint32_t (&m)[8]) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t lo = (t[k] << 16) & 0x7FFF0000u, hi = t[k] & 0x7FFF0000u;
      m[2 * k] = m[2 * k] > lo ? m[2 * k] : lo;
      m[2 * k + 1] = m[2 * k + 1] > hi ? m[2 * k + 1] : hi;
    }
  }
};
template <> struct AbsEach<F16> {
  static constexpr int G = 8;
  static __device__ __forceinline__ void acc(u32x4 t, uint32_t (&m)[8]) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t lo = t[k] & 0x7FFFu, hi = (t[k] >> 16) & 0x7FFFu;
      m[2 * k] = m[2 * k] > lo ? m[2 * k] : lo;
      m[2 * k + 1] = m[2 * k + 1] > hi ? m[2 * k + 1] : hi;
    }
  }
};

__device__ __forceinline__ void emit(float amax, float qmax, float* amax_out, float* scale_out, int64_t idx) {
  if (amax_out) amax_out[idx] = amax;
  if (scale_out) scale_out[idx] = amax / qmax;
}

// row kind: wave `s` (of nb) reduces rows s, s + nb, ... ; VEC: d1 % G == 0 and x 16-byte aligned
template <typename X, bool VEC>
__device__ __forceinline__ void rows_body(const typename X::storage* __restrict__ x, int64_t d0, int64_t d1, int64_t nb,
                                          float qmax, float* __restrict__ amax_out, float* __restrict__ scale_out) {
  using A = AbsBits<X>;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t s = (int64_t(blockIdx.x) * blockDim.x + threadIdx.x) / kWave;
  if (s >= nb) return;                               // whole waves leave together
  uint32_t m = 0;
  for (int64_t row = s; row < d0; row += nb) {
    const typename X::storage* p = x + row * d1;
    if (VEC) {
      const u32x4* pv = reinterpret_cast<const u32x4*>(p);
      const int64_t nvec = d1 / A::kPerVec;
      int64_t v = lane;
      for (; v + 3 * kWave < nvec; v += 4 * kWave) {   // four independent loads in flight
        u32x4 t[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) t[u] = __builtin_nontemporal_load(pv + v + u * kWave);
#pragma unroll
        for (int u = 0; u < 4; ++u) { const uint32_t a = A::of(t[u]); m = m > a ? m : a; }
      }
      for (; v < nvec; v += kWave) { const uint32_t a = A::of(__builtin_nontemporal_load(pv + v)); m = m > a ? m : a; }
    } else {
      // any row length and alignment: the row's whole vectors by 128-bit loads at element alignment (the hardware
      // splits those that straddle a cache line), the d1 % G elements behind them one per lane
      typedef u32x4 u32x4_unaligned __attribute__((aligned(2)));
      const u32x4_unaligned* pv = reinterpret_cast<const u32x4_unaligned*>(p);
      const int64_t nvec = d1 / A::kPerVec;
      int64_t v = lane;
      for (; v + 3 * kWave < nvec; v += 4 * kWave) {
        u32x4 t[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) t[u] = pv[v + u * kWave];
#pragma unroll
        for (int u = 0; u < 4; ++u) { const uint32_t a = A::of(t[u]); m = m > a ? m : a; }
      }
      for (; v < nvec; v += kWave) { const uint32_t a = A::of(pv[v]); m = m > a ? m : a; }
      for (int64_t c = nvec * A::kPerVec + lane; c < d1; c += kWave) { const uint32_t a = A::one(p + c); m = m > a ? m : a; }
    }
  }
  m = wave_reduce(m, MaxU32());
  if (lane == 0) emit(A::finish(m), qmax, amax_out, scale_out, s);
}

// The vector of columns vcol * G .. of row `row` for the column kernels.  UNALIGNED: any d1 and any alignment of x: whole
// vectors by 128-bit loads at element alignment, and the d1 % G columns behind the last whole vector gathered one
// by one into a vector of their own (index d1 / G), zeros in the lanes beyond.
__device__ __forceinline__ uint32_t raw_bits(float v) { return f32_to_bits(v); }
__device__ __forceinline__ uint32_t raw_bits(uint16_t v) { return v; }
template <typename X, bool UNALIGNED>
__device__ __forceinline__ u32x4 column_vector(const typename X::storage* __restrict__ x, int64_t row, int64_t vcol, int64_t d1) {
  constexpr int G = AbsEach<X>::G;
  if (!UNALIGNED) return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(x + row * d1) + vcol);
  typedef u32x4 u32x4_unaligned __attribute__((aligned(2)));
  const typename X::storage* p = x + row * d1 + vcol * G;
  if ((vcol + 1) * G <= d1) return *reinterpret_cast<const u32x4_unaligned*>(p);
  u32x4 t = {0u, 0u, 0u, 0u};
  const int tail = int(d1 - vcol * G);
#pragma unroll
  for (int k = 0; k < G - 1; ++k)
    if (k < tail) {
      if (G == 4) t[k & 3] = raw_bits(p[k]);
      else t[(k >> 1) & 3] |= raw_bits(p[k]) << (16 * (k & 1));
    }
  return t;
}

// col kind, vector form: workgroup = (block b, strip of 64 vectors of columns); wave w takes rows w, w + 4, ... of
// the block, lane l the vector column strip * 64 + l; the four waves' partial maxima meet in LDS.
template <typename X, bool UNALIGNED>
__device__ __forceinline__ void cols_body(const typename X::storage* __restrict__ x, int64_t d0, int64_t d1, int64_t nb,
                                          float qmax, float* __restrict__ amax_out, float* __restrict__ scale_out) {
  using E = AbsEach<X>;
  constexpr int G = E::G;
  __shared__ uint32_t part[4][kWave][G + 1];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int64_t nvec = (d1 + (UNALIGNED ? G - 1 : 0)) / G, strips = (nvec + kWave - 1) / kWave;   // a last partial vector counts when UNALIGNED
  const int64_t b = blockIdx.x / strips, strip = blockIdx.x % strips;
  const int64_t vcol = strip * kWave + lane;
  uint32_t m[G];
#pragma unroll
  for (int k = 0; k < G; ++k) m[k] = 0;
  if (vcol < nvec) {
    const int64_t row0 = b * nb;
    int64_t r = wave;
    for (; r + 12 < nb; r += 16) {                     // four independent loads in flight
      u32x4 t[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) t[u] = column_vector<X, UNALIGNED>(x, row0 + r + 4 * u, vcol, d1);
#pragma unroll
      for (int u = 0; u < 4; ++u) E::acc(t[u], m);
    }
    for (; r < nb; r += 4) E::acc(column_vector<X, UNALIGNED>(x, row0 + r, vcol, d1), m);
  }
#pragma unroll
  for (int k = 0; k < G; ++k) part[wave][lane][k] = m[k];
  __syncthreads();
  if (wave == 0 && vcol < nvec) {
#pragma unroll
    for (int k = 0; k < G; ++k) {
      uint32_t r = part[0][lane][k];
#pragma unroll
      for (int w = 1; w < 4; ++w) r = r > part[w][lane][k] ? r : part[w][lane][k];
      if (vcol * G + k < d1) emit(AbsBits<X>::finish(r), qmax, amax_out, scale_out, b * d1 + vcol * G + k);
    }
  }
}

// col kind, few long blocks (per-channel scales of a [K, N] weight: ONE block of all K rows): the rows of a block are
// dealt to `parts` workgroups, rows [part * rows_per_part, ...), whose column maxima meet in `stage` (one word per
// scale element, zero on entry) through atomic max on the bit patterns; mtrt_amax_finish_* turns the words into
// amax and scale afterwards.  Without the split such a tensor has ceil(d1 / G / 64) workgroups in all.
template <typename X, bool UNALIGNED>
__device__ __forceinline__ void cols_split_body(const typename X::storage* __restrict__ x, int64_t d0, int64_t d1, int64_t nb,
                                                int64_t rows_per_part, uint32_t* __restrict__ stage) {
  using E = AbsEach<X>;
  constexpr int G = E::G;
  __shared__ uint32_t part_max[4][kWave][G + 1];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int64_t nvec = (d1 + (UNALIGNED ? G - 1 : 0)) / G, strips = (nvec + kWave - 1) / kWave;
  const int64_t parts = (nb + rows_per_part - 1) / rows_per_part;
  const int64_t part = blockIdx.x % parts, rest = blockIdx.x / parts;
  const int64_t b = rest / strips, strip = rest % strips;
  const int64_t vcol = strip * kWave + lane;
  const int64_t r0 = part * rows_per_part, r1 = r0 + rows_per_part < nb ? r0 + rows_per_part : nb;
  uint32_t m[G];
#pragma unroll
  for (int k = 0; k < G; ++k) m[k] = 0;
  if (vcol < nvec) {
    const int64_t row0 = b * nb;
    int64_t r = r0 + wave;
    for (; r + 12 < r1; r += 16) {                     // four independent loads in flight
      u32x4 t[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) t[u] = column_vector<X, UNALIGNED>(x, row0 + r + 4 * u, vcol, d1);
#pragma unroll
      for (int u = 0; u < 4; ++u) E::acc(t[u], m);
    }
    for (; r < r1; r += 4) E::acc(column_vector<X, UNALIGNED>(x, row0 + r, vcol, d1), m);
  }
#pragma unroll
  for (int k = 0; k < G; ++k) part_max[wave][lane][k] = m[k];
  __syncthreads();
  if (wave == 0 && vcol < nvec) {
#pragma unroll
    for (int k = 0; k < G; ++k) {
      uint32_t r = part_max[0][lane][k];
#pragma unroll
      for (int w = 1; w < 4; ++w) r = r > part_max[w][lane][k] ? r : part_max[w][lane][k];
      // nobody reads the word before the launch has ended: no ordering, no return value
      if (vcol * G + k < d1) __hip_atomic_fetch_max(stage + b * d1 + vcol * G + k, r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

// row kind, few scales (a channel axis of a few dozen entries in front of large inner extents, or a handful of very
// long rows): one wave per scale leaves the chip empty.  The rows of scale s (s, s + nb, ...) are cut into tiles
// of kRowChunk vectors; `parts` workgroups share the tiles of a scale (workgroup s * parts + p the p-th range of
// them, its four waves one tile at a time) and meet in stage[s] (zero on entry) by atomic max, one per workgroup;
// mtrt_amax_finish_* follows.  d1 % G == 0, x 16-byte aligned.
constexpr int kRowChunk = 1024;                      // vectors per tile: 16 per lane, four loads in flight at a time

template <typename X>
__device__ __forceinline__ void rows_split_body(const typename X::storage* __restrict__ x, int64_t d0, int64_t d1, int64_t nb,
                                                int64_t parts, uint32_t* __restrict__ stage) {
  using A = AbsBits<X>;
  __shared__ uint32_t wave_max[4];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int64_t s = blockIdx.x / parts, p = blockIdx.x % parts;
  const int64_t nvec = d1 / A::kPerVec, chunks = (nvec + kRowChunk - 1) / kRowChunk;
  const int64_t rows_s = (d0 - s + nb - 1) / nb;     // rows s, s + nb, ... below d0
  const int64_t tiles = rows_s * chunks;
  const int64_t t0 = tiles * p / parts, t1 = tiles * (p + 1) / parts;
  uint32_t m = 0;
  for (int64_t t = t0 + wave; t < t1; t += 4) {
    const int64_t i = t / chunks, c = t - i * chunks;
    const u32x4* pv = reinterpret_cast<const u32x4*>(x + (s + i * nb) * d1);
    const int64_t v1 = (c + 1) * kRowChunk < nvec ? (c + 1) * kRowChunk : nvec;
    int64_t v = c * kRowChunk + lane;
    for (; v + 3 * kWave < v1; v += 4 * kWave) {       // four independent loads in flight
      u32x4 tt[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) tt[u] = __builtin_nontemporal_load(pv + v + u * kWave);
#pragma unroll
      for (int u = 0; u < 4; ++u) { const uint32_t a = A::of(tt[u]); m = m > a ? m : a; }
    }
    for (; v < v1; v += kWave) { const uint32_t a = A::of(__builtin_nontemporal_load(pv + v)); m = m > a ? m : a; }
  }
  m = wave_reduce(m, MaxU32());
  if (lane == 0) wave_max[wave] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t r = wave_max[0];
#pragma unroll
    for (int w = 1; w < 4; ++w) r = r > wave_max[w] ? r : wave_max[w];
    // nobody reads the word before the launch has ended: no ordering, no return value
    __hip_atomic_fetch_max(stage + s, r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// stage word (maximum bit pattern) -> amax and scale; `stage` may be amax_out or scale_out itself
template <typename X>
__device__ __forceinline__ void finish_body(const uint32_t* stage, int64_t count, float qmax, float* amax_out, float* scale_out) {
  const int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= count) return;
  emit(AbsBits<X>::finish(stage[i]), qmax, amax_out, scale_out, i);
}

// col kind, any shape: one lane per (block, column)
template <typename X>
__device__ __forceinline__ void cols_any_body(const typename X::storage* __restrict__ x, int64_t d0, int64_t d1, int64_t nb,
                                              float qmax, float* __restrict__ amax_out, float* __restrict__ scale_out) {
  using A = AbsBits<X>;
  const int64_t total = (d0 / nb) * d1;
  for (int64_t e = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; e < total; e += int64_t(gridDim.x) * blockDim.x) {
    const int64_t b = e / d1, c = e - b * d1;
    uint32_t m = 0;
    for (int64_t r = 0; r < nb; ++r) { const uint32_t a = A::one(x + (b * nb + r) * d1 + c); m = m > a ? m : a; }
    emit(A::finish(m), qmax, amax_out, scale_out, e);
  }
}

}  // namespace amax_scales_cluster

// (x, d0, d1, nb, qmax, amax_out or null, scale_out or null)
//   rows / rows_any : grid = ceil(nb / 4), block = 256 (one wave per scale)
//   cols            : grid = (d0 / nb) * ceil(d1 / G / 64), block = 256 ; d1 % G == 0, x 16-byte aligned
//   cols_u, cols_split_u : the same two for any d1 and alignment, grid with ceil(d1 / G) vectors per row
//   cols_any        : grid-stride, block = 256
// (x, d0, d1, nb, parts, stage) rows_split : grid = nb * parts, block = 256 ; stage = nb zeroed words ; then finish
// (x, d0, d1, nb, rows_per_part, stage) cols_split : grid = (d0 / nb) * ceil(d1 / G / 64) * ceil(nb / rows_per_part),
//   block = 256 ; stage = (d0 / nb) * d1 zeroed words ; then (stage, count, qmax, amax_out or null, scale_out or null)
//   finish : grid = ceil(count / 256), block = 256
#define MTRT_AMAX_SCALES_KERNELS(XN, XT)                                                                              \
  extern "C" __global__ void __launch_bounds__(256) mtrt_amax_rows_##XN(                                               \
      const XT::storage* x, int64_t d0, int64_t d1, int64_t nb, float qmax, float* amax_out, float* scale_out) {       \
    amax_scales_cluster::rows_body<XT, true>(x, d0, d1, nb, qmax, amax_out, scale_out); }                              \
  extern "C" __global__ void __launch_bounds__(256) mtrt_amax_rows_any_##XN(                                           \
      const XT::storage* x, int64_t d0, int64_t d1, int64_t nb, float qmax, float* amax_out, float* scale_out) {       \
    amax_scales_cluster::rows_body<XT, false>(x, d0, d1, nb, qmax, amax_out, scale_out); }                             \
  extern "C" __global__ void __launch_bounds__(256) mtrt_amax_cols_##XN(                                               \
      const XT::storage* x, int64_t d0, int64_t d1, int64_t nb, float qmax, float* amax_out, float* scale_out) {       \
    amax_scales_cluster::cols_body<XT, false>(x, d0, d1, nb, qmax, amax_out, scale_out); }                             \
  extern "C" __global__ void __launch_bounds__(256) mtrt_amax_cols_u_##XN(                                             \
      const XT::storage* x, int64_t d0, int64_t d1, int64_t nb, float qmax, float* amax_out, float* scale_out) {       \
    amax_scales_cluster::cols_body<XT, true>(x, d0, d1, nb, qmax, amax_out, scale_out); }                              \
  extern "C" __global__ void __launch_bounds__(256) mtrt_amax_cols_split_##XN(                                         \
      const XT::storage* x, int64_t d0, int64_t d1, int64_t nb, int64_t rows_per_part, uint32_t* stage) {              \
    amax_scales_cluster::cols_split_body<XT, false>(x, d0, d1, nb, rows_per_part, stage); }                            \
  extern "C" __global__ void __launch_bounds__(256) mtrt_amax_cols_split_u_##XN(                                       \
      const XT::storage* x, int64_t d0, int64_t d1, int64_t nb, int64_t rows_per_part, uint32_t* stage) {              \
    amax_scales_cluster::cols_split_body<XT, true>(x, d0, d1, nb, rows_per_part, stage); }                             \
  extern "C" __global__ void __launch_bounds__(256) mtrt_amax_rows_split_##XN(                                         \
      const XT::storage* x, int64_t d0, int64_t d1, int64_t nb, int64_t parts, uint32_t* stage) {                      \
    amax_scales_cluster::rows_split_body<XT>(x, d0, d1, nb, parts, stage); }                                           \
  extern "C" __global__ void __launch_bounds__(256) mtrt_amax_finish_##XN(                                             \
      const uint32_t* stage, int64_t count, float qmax, float* amax_out, float* scale_out) {                           \
    amax_scales_cluster::finish_body<XT>(stage, count, qmax, amax_out, scale_out); }                                   \
  extern "C" __global__ void __launch_bounds__(256) mtrt_amax_cols_any_##XN(                                           \
      const XT::storage* x, int64_t d0, int64_t d1, int64_t nb, float qmax, float* amax_out, float* scale_out) {       \
    amax_scales_cluster::cols_any_body<XT>(x, d0, d1, nb, qmax, amax_out, scale_out); }
MTRT_AMAX_SCALES_KERNELS(f32, F32)
MTRT_AMAX_SCALES_KERNELS(f16, F16)
MTRT_AMAX_SCALES_KERNELS(bf16, BF16)
