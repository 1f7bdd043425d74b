// Fused elementwise+reduce clusters over the last dimension: LayerNorm and softmax.
//
// LayerNorm (the decomposition the reference recognises,
//   mlir-tensorrt/tensorrt/lib/TensorRT/Transforms/RaiseNormalizations.pdll:277-308;
//   user API tripy/nvtripy/frontend/module/layernorm.py:30-70):
//     xf = f32(x); mu = sum(xf)/D; d = xf - mu; var = sum(d*d)/D;
//     y = narrow(((d * (1/sqrt(var + eps))) * f32(gamma)) + f32(beta))
// softmax (mlir-tensorrt/compiler/lib/Dialect/StablehloExt/Utils/StablehloMatchers.cpp:311-335;
//   tripy/nvtripy/frontend/ops/softmax.py:30-82):
//     xf = f32(x); m = max(xf); e = exp(xf - m); s = sum(e); y = narrow(e / s)   [computed as e * (1/s)]
//
// The reference's code generator emits at least three (LayerNorm) or four (softmax)
// kernels for these, each re-reading the tensor, with one thread walking a whole
// row (mlir-tensorrt/kernel/lib/Utils/TilingUtils.cpp:669-677).  Here each row is
// read from HBM exactly once: ONE WAVE OWNS ONE ROW, the row lives in that wave's
// registers (NV 128-bit vectors per lane, lane l holding vectors l, l+64, ...: every
// load instruction of the wave covers 1 KiB of contiguous HBM), and both row
// reductions are cross-lane exchanges with no LDS and no barrier.  Longer rows (up to
// 1024 * 16 vectors) are owned by a workgroup in the same way ("_g" kernels); rows that
// fit neither scheme (D not a multiple of the vector width, or longer still) use the
// workgroup-per-row "_any" kernels, which re-read the row from cache.
//
// All arithmetic is f32 with the operation order above; reductions are trees
// rather than the host's left-to-right sums, which the float tolerance covers.
#include "common.hpp"

using namespace mtrt_dev;

namespace norm_cluster {

constexpr int kNormThreads = 256;
constexpr int kRowsPerBlock = kNormThreads / kWave;

template <typename X> struct Vec;     // one 128-bit vector <-> floats
template <> struct Vec<F32> {
  static constexpr int kElems = 4;
  static __device__ __forceinline__ void unpack(u32x4 t, float* v) {
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = bits_to_f32(t[j]);
  }
  static __device__ __forceinline__ u32x4 pack(const float* v) {
    u32x4 t;
#pragma unroll
    for (int j = 0; j < 4; ++j) t[j] = f32_to_bits(v[j]);
    return t;
  }
};
template <> struct Vec<BF16> {
  static constexpr int kElems = 8;
  static __device__ __forceinline__ void unpack(u32x4 t, float* v) {
#pragma unroll
    for (int j = 0; j < 4; ++j) { v[2 * j] = bits_to_f32(t[j] << 16); v[2 * j + 1] = bits_to_f32(t[j] & 0xFFFF0000u); }
  }
  static __device__ __forceinline__ u32x4 pack(const float* v) {
    u32x4 t;
#pragma unroll
    for (int j = 0; j < 4; ++j) t[j] = f32_to_bf16_bits(v[2 * j]) | (f32_to_bf16_bits(v[2 * j + 1]) << 16);
    return t;
  }
};
template <> struct Vec<F16> {
  static constexpr int kElems = 8;
  static __device__ __forceinline__ void unpack(u32x4 t, float* v) {
#pragma unroll
    for (int j = 0; j < 4; ++j) { v[2 * j] = f16_bits_to_f32(t[j] & 0xFFFFu); v[2 * j + 1] = f16_bits_to_f32(t[j] >> 16); }
  }
  static __device__ __forceinline__ u32x4 pack(const float* v) {
    u32x4 t;
#pragma unroll
    for (int j = 0; j < 4; ++j) t[j] = f32_to_f16_bits(v[2 * j]) | (f32_to_f16_bits(v[2 * j + 1]) << 16);
    return t;
  }
};

// Load the wave's row into registers: NV vectors per lane.  Every lane always loads (vectors past
// the end of the row re-read the row's last vector and are replaced by `fill` afterwards), so the
// loads are issued back to back with no branches between them; with FULL (the row fills all
// 64 * NV vectors) the replacement disappears as well.
template <typename X, int NV, bool FULL>
__device__ __forceinline__ void load_row(const u32x4* __restrict__ row, int nvec, int lane, float fill,
                                         float (&v)[NV * Vec<X>::kElems]) {
  constexpr int E = Vec<X>::kElems;
  u32x4 t[NV];
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int idx = lane + kWave * j;
    t[j] = __builtin_nontemporal_load(row + (FULL ? idx : min(idx, nvec - 1)));
  }
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    Vec<X>::unpack(t[j], &v[j * E]);
    if (!FULL) {
      const bool live = lane + kWave * j < nvec;
#pragma unroll
      for (int k = 0; k < E; ++k) v[j * E + k] = live ? v[j * E + k] : fill;
    }
  }
}

// Hides a vector's provenance from the optimiser (no instruction is emitted).
__device__ __forceinline__ void opaque(u32x4& t) { __asm__ volatile("" : "+v"(t)); }

// The row stays in registers in its STORAGE form (NV 128-bit vectors per lane) and is widened
// again in each of the three passes: for 16-bit types that halves the live registers compared
// with keeping f32 values (a widening is one shift or mask per element), and the higher
// occupancy it buys is worth more to this memory-bound kernel than the extra VALU work.
template <typename X, int NV, bool FULL>
__device__ __forceinline__ void layernorm_row(const typename X::storage* __restrict__ x,
                                              const typename X::storage* __restrict__ gamma,
                                              const typename X::storage* __restrict__ beta,
                                              typename X::storage* __restrict__ y, int64_t row, int64_t d, float eps) {
  constexpr int E = Vec<X>::kElems;
  const int lane = threadIdx.x & (kWave - 1);
  const int nvec = int(d / E);
  const u32x4* xr = reinterpret_cast<const u32x4*>(x + row * d);
  u32x4 t[NV];
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int idx = lane + kWave * j;
    t[j] = __builtin_nontemporal_load(xr + (FULL ? idx : min(idx, nvec - 1)));
  }

  const float fd = float(d);
  float sum = 0.0f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const bool live = FULL || lane + kWave * j < nvec;
    float v[E];
    Vec<X>::unpack(t[j], v);
#pragma unroll
    for (int k = 0; k < E; ++k) sum = sum + (live ? v[k] : 0.0f);
  }
  const float mu = wave_reduce(sum, SumF32()) / fd;
  float sq = 0.0f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const bool live = FULL || lane + kWave * j < nvec;
    float v[E];
    opaque(t[j]);                                    // widen again instead of keeping pass 1's values live
    Vec<X>::unpack(t[j], v);
#pragma unroll
    for (int k = 0; k < E; ++k) {
      const float dv = v[k] - mu;
      sq = sq + (live ? dv * dv : 0.0f);
    }
  }
  const float var = wave_reduce(sq, SumF32()) / fd;
  const float rstd = 1.0f / sqrtf(var + eps);

  const u32x4* gv = reinterpret_cast<const u32x4*>(gamma);
  const u32x4* bv = reinterpret_cast<const u32x4*>(beta);
  u32x4* yr = reinterpret_cast<u32x4*>(y + row * d);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int idx = lane + kWave * j;
    const int idc = FULL ? idx : min(idx, nvec - 1);
    float v[E], g[E], b[E], o[E];
    opaque(t[j]);
    Vec<X>::unpack(t[j], v);
    Vec<X>::unpack(gv[idc], g);
    Vec<X>::unpack(bv[idc], b);
#pragma unroll
    for (int k = 0; k < E; ++k) o[k] = (((v[k] - mu) * rstd) * g[k]) + b[k];
    if (FULL || idx < nvec) __builtin_nontemporal_store(Vec<X>::pack(o), yr + idx);
  }
}

template <typename X, int NV>
__device__ __forceinline__ void layernorm_rows(const typename X::storage* __restrict__ x,
                                               const typename X::storage* __restrict__ gamma,
                                               const typename X::storage* __restrict__ beta,
                                               typename X::storage* __restrict__ y, int64_t rows, int64_t d, float eps) {
  // the wave index as a scalar: the row pointers are then wave-uniform and the accesses need one lane offset, not an address pair each
  const int64_t row = int64_t(blockIdx.x) * kRowsPerBlock + __builtin_amdgcn_readfirstlane(int(threadIdx.x / kWave));
  if (row >= rows) return;                           // whole wave leaves together
  if (d == int64_t(Vec<X>::kElems) * kWave * NV)
    layernorm_row<X, NV, true>(x, gamma, beta, y, row, d, eps);
  else
    layernorm_row<X, NV, false>(x, gamma, beta, y, row, d, eps);
}

template <typename X, int NV, bool FULL>
__device__ __forceinline__ void softmax_row(const typename X::storage* __restrict__ x, typename X::storage* __restrict__ y,
                                            int64_t row, int64_t d) {
  constexpr int E = Vec<X>::kElems;
  const int lane = threadIdx.x & (kWave - 1);
  const int nvec = int(d / E);
  const u32x4* xr = reinterpret_cast<const u32x4*>(x + row * d);
  float v[NV * E];
  load_row<X, NV, FULL>(xr, nvec, lane, -INFINITY, v);

  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < NV * E; ++i) mx = fmaxf(mx, v[i]);
  mx = wave_reduce(mx, MaxF32());
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < NV * E; ++i) {
    v[i] = __expf(v[i] - mx);                        // exp(-inf) = 0 for the fill lanes
    s = s + v[i];
  }
  s = wave_reduce(s, SumF32());
  // e / s as e * (1/s): one correctly rounded reciprocal per row instead of a divide per element; at most one
  // f32 ulp from the quotient.  Together with the hardware exponential (2^(d * log2 e), a few f32 ulps off for
  // |d| ~ 10) that is far below what the order of the row sum already changes: with an exponential good to one
  // ulp and a remainder-corrected quotient the share of f16 outputs that differ from the host's by one ulp
  // stayed at 0.05 % (4096 x 4096, sigma 2) and the launch took 1 us longer, so the short forms are kept.
  const float inv = 1.0f / s;
  u32x4* yr = reinterpret_cast<u32x4*>(y + row * d);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int idx = lane + kWave * j;
    float o[E];
#pragma unroll
    for (int k = 0; k < E; ++k) o[k] = v[j * E + k] * inv;
    if (FULL || idx < nvec) __builtin_nontemporal_store(Vec<X>::pack(o), yr + idx);
  }
}

template <typename X, int NV>
__device__ __forceinline__ void softmax_rows(const typename X::storage* __restrict__ x, typename X::storage* __restrict__ y,
                                             int64_t rows, int64_t d) {
  // the wave index as a scalar: the row pointers are then wave-uniform and the accesses need one lane offset, not an address pair each
  const int64_t row = int64_t(blockIdx.x) * kRowsPerBlock + __builtin_amdgcn_readfirstlane(int(threadIdx.x / kWave));
  if (row >= rows) return;
  if (d == int64_t(Vec<X>::kElems) * kWave * NV)
    softmax_row<X, NV, true>(x, y, row, d);
  else
    softmax_row<X, NV, false>(x, y, row, d);
}

// ---- rows longer than one wave's registers, and rows of any length or alignment: a GROUP of lanes owns one row ----
// THREADS lanes hold the row, NV vectors each (lane l the vectors l, l + THREADS, ...), in storage form; the row
// reductions are a cross-lane exchange per wave and, when the group is a whole workgroup (256 or 1024 lanes), a
// meeting of the waves' values in LDS.  The row is still read from HBM exactly once.  Workgroup-sized groups
// cover 64 * 16 < D / E <= 1024 * 16 vectors (hidden sizes above 8192, vocabulary-sized softmax rows).
// RAGGED: D need not be a multiple of the vector width E and nothing need be 16-byte aligned: the D / E whole
// vectors of a row are moved by 128-bit accesses at element alignment (the hardware splits those that straddle
// a line), the D % E elements behind them one each by the group's first lanes.  With THREADS = 64 that is the
// one-wave-per-row scheme for rows such as 197, 1500 or 50257 elements.
template <bool RAGGED> struct RowVector { typedef u32x4 type; };
template <> struct RowVector<true> { typedef u32x4 type __attribute__((aligned(2))); };

template <int THREADS, typename Op>
__device__ __forceinline__ float group_reduce(float v, Op op, float* lds) {
  if (THREADS < kWave) {                             // several rows per wave: exchanges stay inside the row's lanes
#pragma unroll
    for (int off = THREADS / 2; off > 0; off >>= 1) v = op(v, __shfl_xor(v, off, kWave));
    return v;
  }
  v = wave_reduce(v, op);
  if (THREADS == kWave) return v;
  __syncthreads();                                   // lds may still be read from the previous reduction
  if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = v;
  __syncthreads();
  float r = lds[0];
#pragma unroll
  for (int w = 1; w < THREADS / kWave; ++w) r = op(r, lds[w]);
  return r;                                          // the same value, combined in the same order, in every lane
}

template <typename X, int NV, int THREADS, bool FULL, bool RAGGED>
__device__ __forceinline__ void layernorm_group_row(const typename X::storage* __restrict__ x,
                                                    const typename X::storage* __restrict__ gamma,
                                                    const typename X::storage* __restrict__ beta,
                                                    typename X::storage* __restrict__ y, int64_t row, int64_t d, float eps,
                                                    float* lds) {
  constexpr int E = Vec<X>::kElems;
  using V = typename RowVector<RAGGED>::type;
  const int lane = int(threadIdx.x) & (THREADS - 1);
  const int nvec = int(d / E), tail = RAGGED ? int(d - int64_t(nvec) * E) : 0;
  const V* xr = reinterpret_cast<const V*>(x + row * d);
  u32x4 t[NV];
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int idx = lane + THREADS * j;
    if (RAGGED && nvec == 0) t[j] = (u32x4){0u, 0u, 0u, 0u};   // a row shorter than one vector: only the scalar elements below
    else t[j] = __builtin_nontemporal_load(xr + (FULL ? idx : min(idx, nvec - 1)));
  }
  const bool extra = RAGGED && lane < tail;          // this lane also owns element nvec * E + lane
  const int64_t ec = int64_t(nvec) * E + lane;
  const float xe = extra ? Tile<X>::load1(x + row * d + ec) : 0.0f;
  const float fd = float(d);
  float sum = xe;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const bool live = FULL || lane + THREADS * j < nvec;
    float v[E];
    Vec<X>::unpack(t[j], v);
#pragma unroll
    for (int k = 0; k < E; ++k) sum = sum + (live ? v[k] : 0.0f);
  }
  const float mu = group_reduce<THREADS>(sum, SumF32(), lds) / fd;
  float sq = extra ? (xe - mu) * (xe - mu) : 0.0f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const bool live = FULL || lane + THREADS * j < nvec;
    float v[E];
    opaque(t[j]);                                    // widen again instead of keeping pass 1's values live
    Vec<X>::unpack(t[j], v);
#pragma unroll
    for (int k = 0; k < E; ++k) {
      const float dv = v[k] - mu;
      sq = sq + (live ? dv * dv : 0.0f);
    }
  }
  const float var = group_reduce<THREADS>(sq, SumF32(), lds) / fd;
  const float rstd = 1.0f / sqrtf(var + eps);
  const V* gv = reinterpret_cast<const V*>(gamma);
  const V* bv = reinterpret_cast<const V*>(beta);
  V* yr = reinterpret_cast<V*>(y + row * d);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int idx = lane + THREADS * j;
    const int idc = FULL ? idx : min(idx, nvec - 1);
    if (RAGGED && nvec == 0) continue;               // no whole vector: nothing to read or store here
    float v[E], g[E], b[E], o[E];
    opaque(t[j]);
    Vec<X>::unpack(t[j], v);
    Vec<X>::unpack(gv[idc], g);
    Vec<X>::unpack(bv[idc], b);
#pragma unroll
    for (int k = 0; k < E; ++k) o[k] = (((v[k] - mu) * rstd) * g[k]) + b[k];
    if (FULL || idx < nvec) __builtin_nontemporal_store(Vec<X>::pack(o), yr + idx);
  }
  if (extra)
    Tile<X>::store1(y + row * d + ec, (((xe - mu) * rstd) * Tile<X>::load1(gamma + ec)) + Tile<X>::load1(beta + ec));
}

// The group's row: a workgroup-sized group takes row blockIdx.x, wave-sized groups the rows 4 * blockIdx.x + wave,
// groups of 8, 16 or 32 lanes (short rows, several to a wave) the rows (256 / THREADS) * blockIdx.x + group.
template <int THREADS>
__device__ __forceinline__ int64_t group_row() {
  if (THREADS == kWave)
    return int64_t(blockIdx.x) * kRowsPerBlock + __builtin_amdgcn_readfirstlane(int(threadIdx.x / kWave));
  if (THREADS < kWave)
    return int64_t(blockIdx.x) * (kNormThreads / THREADS) + int(threadIdx.x) / THREADS;
  return blockIdx.x;
}

template <typename X, int NV, int THREADS, bool RAGGED>
__device__ __forceinline__ void layernorm_group(const typename X::storage* __restrict__ x,
                                                const typename X::storage* __restrict__ gamma,
                                                const typename X::storage* __restrict__ beta,
                                                typename X::storage* __restrict__ y, int64_t rows, int64_t d, float eps) {
  __shared__ float lds[THREADS >= kWave ? THREADS / kWave : 1];
  const int64_t row = group_row<THREADS>();
  if (row >= rows) return;                           // groups of a wave or less only (no barrier follows there); grid = rows otherwise
  if (!RAGGED && d == int64_t(Vec<X>::kElems) * THREADS * NV)
    layernorm_group_row<X, NV, THREADS, true, false>(x, gamma, beta, y, row, d, eps, lds);
  else
    layernorm_group_row<X, NV, THREADS, false, RAGGED>(x, gamma, beta, y, row, d, eps, lds);
}

// KEEP: the exponentials stay in registers (f32) between the sum and the output pass; without it they are
// computed again from the stored row (the 1024-lane form has 128 registers per lane, not enough for both).
template <typename X, int NV, int THREADS, bool FULL, bool KEEP, bool RAGGED>
__device__ __forceinline__ void softmax_group_row(const typename X::storage* __restrict__ x, typename X::storage* __restrict__ y,
                                                  int64_t row, int64_t d, float* lds) {
  constexpr int E = Vec<X>::kElems;
  using V = typename RowVector<RAGGED>::type;
  const int lane = int(threadIdx.x) & (THREADS - 1);
  const int nvec = int(d / E), tail = RAGGED ? int(d - int64_t(nvec) * E) : 0;
  const V* xr = reinterpret_cast<const V*>(x + row * d);
  u32x4 t[NV];
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int idx = lane + THREADS * j;
    if (RAGGED && nvec == 0) t[j] = (u32x4){0u, 0u, 0u, 0u};   // a row shorter than one vector: only the scalar elements below
    else t[j] = __builtin_nontemporal_load(xr + (FULL ? idx : min(idx, nvec - 1)));
  }
  const bool extra = RAGGED && lane < tail;          // this lane also owns element nvec * E + lane
  const int64_t ec = int64_t(nvec) * E + lane;
  const float xe = extra ? Tile<X>::load1(x + row * d + ec) : -INFINITY;
  float mx = xe;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const bool live = FULL || lane + THREADS * j < nvec;
    float v[E];
    Vec<X>::unpack(t[j], v);
#pragma unroll
    for (int k = 0; k < E; ++k) mx = fmaxf(mx, live ? v[k] : -INFINITY);
  }
  mx = group_reduce<THREADS>(mx, MaxF32(), lds);
  float e[KEEP ? NV * E : 1];
  const float ee = extra ? __expf(xe - mx) : 0.0f;
  float s = ee;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const bool live = FULL || lane + THREADS * j < nvec;
    float v[E];
    opaque(t[j]);
    Vec<X>::unpack(t[j], v);
#pragma unroll
    for (int k = 0; k < E; ++k) {
      const float ev = live ? __expf(v[k] - mx) : 0.0f;
      if (KEEP) e[j * E + k] = ev;
      s = s + ev;
    }
  }
  s = group_reduce<THREADS>(s, SumF32(), lds);
  const float inv = 1.0f / s;                         // e * (1/s), as in softmax_row
  V* yr = reinterpret_cast<V*>(y + row * d);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int idx = lane + THREADS * j;
    float o[E];
    if (KEEP) {
#pragma unroll
      for (int k = 0; k < E; ++k) o[k] = e[j * E + k] * inv;
    } else {
      float v[E];
      opaque(t[j]);
      Vec<X>::unpack(t[j], v);
#pragma unroll
      for (int k = 0; k < E; ++k) o[k] = __expf(v[k] - mx) * inv;
    }
    if (FULL || idx < nvec) __builtin_nontemporal_store(Vec<X>::pack(o), yr + idx);
  }
  if (extra) Tile<X>::store1(y + row * d + ec, ee * inv);
}

template <typename X, int NV, int THREADS, bool RAGGED>
__device__ __forceinline__ void softmax_group(const typename X::storage* __restrict__ x, typename X::storage* __restrict__ y,
                                              int64_t rows, int64_t d) {
  __shared__ float lds[THREADS >= kWave ? THREADS / kWave : 1];
  constexpr bool kKeep = THREADS <= 256;
  const int64_t row = group_row<THREADS>();
  if (row >= rows) return;                           // groups of a wave or less only (no barrier follows there); grid = rows otherwise
  if (!RAGGED && d == int64_t(Vec<X>::kElems) * THREADS * NV)
    softmax_group_row<X, NV, THREADS, true, kKeep, false>(x, y, row, d, lds);
  else
    softmax_group_row<X, NV, THREADS, false, kKeep, RAGGED>(x, y, row, d, lds);
}

// ---- any D, any alignment: one workgroup per row, row re-read from cache -------------
template <typename Op>
__device__ __forceinline__ float block_reduce(float v, Op op, float* lds) {
  v = wave_reduce(v, op);
  const int wave = threadIdx.x / kWave;
  __syncthreads();                                   // lds may still be read from the previous round
  if ((threadIdx.x & (kWave - 1)) == 0) lds[wave] = v;
  __syncthreads();
  float r = lds[0];
#pragma unroll
  for (int w = 1; w < kNormThreads / kWave; ++w) r = op(r, lds[w]);
  return r;
}

// Rows of any length and alignment: whole vectors by 128-bit accesses at element alignment, the d % E elements behind
// them one per lane; the row is read three times (the second and third time from cache).
template <typename X>
__device__ __forceinline__ void layernorm_any(const typename X::storage* __restrict__ x,
                                              const typename X::storage* __restrict__ gamma,
                                              const typename X::storage* __restrict__ beta,
                                              typename X::storage* __restrict__ y, int64_t rows, int64_t d, float eps) {
  constexpr int E = Vec<X>::kElems;
  using V = typename RowVector<true>::type;
  __shared__ float lds[kNormThreads / kWave];
  const int64_t nvec = d / E, tail0 = nvec * E;
  const V* gv = reinterpret_cast<const V*>(gamma);
  const V* bv = reinterpret_cast<const V*>(beta);
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const typename X::storage* xr = x + row * d;
    const V* xv = reinterpret_cast<const V*>(xr);
    float sum = 0.0f;
    for (int64_t v = threadIdx.x; v < nvec; v += kNormThreads) {
      float f[E];
      Vec<X>::unpack(xv[v], f);
#pragma unroll
      for (int k = 0; k < E; ++k) sum = sum + f[k];
    }
    for (int64_t c = tail0 + threadIdx.x; c < d; c += kNormThreads) sum = sum + Tile<X>::load1(xr + c);
    const float mu = block_reduce(sum, SumF32(), lds) / float(d);
    float sq = 0.0f;
    for (int64_t v = threadIdx.x; v < nvec; v += kNormThreads) {
      float f[E];
      Vec<X>::unpack(xv[v], f);
#pragma unroll
      for (int k = 0; k < E; ++k) { const float dv = f[k] - mu; sq = sq + dv * dv; }
    }
    for (int64_t c = tail0 + threadIdx.x; c < d; c += kNormThreads) { const float dv = Tile<X>::load1(xr + c) - mu; sq = sq + dv * dv; }
    const float var = block_reduce(sq, SumF32(), lds) / float(d);
    const float rstd = 1.0f / sqrtf(var + eps);
    V* yv = reinterpret_cast<V*>(y + row * d);
    for (int64_t v = threadIdx.x; v < nvec; v += kNormThreads) {
      float f[E], g[E], b[E], o[E];
      Vec<X>::unpack(xv[v], f);
      Vec<X>::unpack(gv[v], g);
      Vec<X>::unpack(bv[v], b);
#pragma unroll
      for (int k = 0; k < E; ++k) o[k] = (((f[k] - mu) * rstd) * g[k]) + b[k];
      yv[v] = Vec<X>::pack(o);
    }
    for (int64_t c = tail0 + threadIdx.x; c < d; c += kNormThreads) {
      const float dv = Tile<X>::load1(xr + c) - mu;
      Tile<X>::store1(y + row * d + c, ((dv * rstd) * Tile<X>::load1(gamma + c)) + Tile<X>::load1(beta + c));
    }
  }
}

template <typename X>
__device__ __forceinline__ void softmax_any(const typename X::storage* __restrict__ x, typename X::storage* __restrict__ y,
                                            int64_t rows, int64_t d) {
  constexpr int E = Vec<X>::kElems;
  using V = typename RowVector<true>::type;
  __shared__ float lds[kNormThreads / kWave];
  const int64_t nvec = d / E, tail0 = nvec * E;
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const typename X::storage* xr = x + row * d;
    const V* xv = reinterpret_cast<const V*>(xr);
    float mx = -INFINITY;
    for (int64_t v = threadIdx.x; v < nvec; v += kNormThreads) {
      float f[E];
      Vec<X>::unpack(xv[v], f);
#pragma unroll
      for (int k = 0; k < E; ++k) mx = fmaxf(mx, f[k]);
    }
    for (int64_t c = tail0 + threadIdx.x; c < d; c += kNormThreads) mx = fmaxf(mx, Tile<X>::load1(xr + c));
    mx = block_reduce(mx, MaxF32(), lds);
    float s = 0.0f;
    for (int64_t v = threadIdx.x; v < nvec; v += kNormThreads) {
      float f[E];
      Vec<X>::unpack(xv[v], f);
#pragma unroll
      for (int k = 0; k < E; ++k) s = s + __expf(f[k] - mx);
    }
    for (int64_t c = tail0 + threadIdx.x; c < d; c += kNormThreads) s = s + __expf(Tile<X>::load1(xr + c) - mx);
    s = block_reduce(s, SumF32(), lds);
    const float inv = 1.0f / s;
    V* yv = reinterpret_cast<V*>(y + row * d);
    for (int64_t v = threadIdx.x; v < nvec; v += kNormThreads) {
      float f[E], o[E];
      Vec<X>::unpack(xv[v], f);
#pragma unroll
      for (int k = 0; k < E; ++k) o[k] = __expf(f[k] - mx) * inv;
      yv[v] = Vec<X>::pack(o);
    }
    for (int64_t c = tail0 + threadIdx.x; c < d; c += kNormThreads)
      Tile<X>::store1(y + row * d + c, __expf(Tile<X>::load1(xr + c) - mx) * inv);
  }
}

}  // namespace norm_cluster
using namespace norm_cluster;

// _v8r: the eight-vector LayerNorm held to 64 registers, eight waves per SIMD.  It is the slower kernel per
// row (the affine parameters are fetched one vector at a time), but when the whole tensor then fits on the
// chip at once while the default kernel (five waves per SIMD) would need a second, partly filled round, the
// launch is one read phase followed by one write phase and ends sooner (bf16 [8192, 4096]: 26.6 -> 24.3 us;
// [4096, 4096] 11.3 -> 12.7 us and [16384, 4096] 47.4 -> 50.4 us, hence only inside that window).
// Entry points.  mtrt_layernorm_<t>_v<NV>(x, gamma, beta, y, rows, d, eps)
//                mtrt_softmax_<t>_v<NV>(x, y, rows, d)         NV = vectors per lane
#define MTRT_LN_OCCUPANCY_1
#define MTRT_LN_OCCUPANCY_2
#define MTRT_LN_OCCUPANCY_4
#define MTRT_LN_OCCUPANCY_8 __attribute__((amdgpu_waves_per_eu(5, 5)))
#define MTRT_LN_OCCUPANCY_16
#define MTRT_NORM_KERNELS(XN, XT, NV)                                                                         \
  extern "C" __global__ void __launch_bounds__(kNormThreads) MTRT_LN_OCCUPANCY_##NV mtrt_layernorm_##XN##_v##NV(                      \
      const XT::storage* x, const XT::storage* gamma, const XT::storage* beta, XT::storage* y, int64_t rows,  \
      int64_t d, float eps) { layernorm_rows<XT, NV>(x, gamma, beta, y, rows, d, eps); }                      \
  extern "C" __global__ void __launch_bounds__(kNormThreads) mtrt_softmax_##XN##_v##NV(                        \
      const XT::storage* x, XT::storage* y, int64_t rows, int64_t d) { softmax_rows<XT, NV>(x, y, rows, d); }

#define MTRT_NORM_FOR_TYPE(XN, XT)                                                                            \
  MTRT_NORM_KERNELS(XN, XT, 1) MTRT_NORM_KERNELS(XN, XT, 2) MTRT_NORM_KERNELS(XN, XT, 4)                       \
  MTRT_NORM_KERNELS(XN, XT, 8) MTRT_NORM_KERNELS(XN, XT, 16)                                                   \
  extern "C" __global__ void __launch_bounds__(kNormThreads) __attribute__((amdgpu_waves_per_eu(8, 8)))        \
  mtrt_layernorm_##XN##_v8r(const XT::storage* x, const XT::storage* gamma, const XT::storage* beta,           \
                            XT::storage* y, int64_t rows, int64_t d, float eps) {                              \
    layernorm_rows<XT, 8>(x, gamma, beta, y, rows, d, eps);                                                    \
  }                                                                                                            \
  extern "C" __global__ void __launch_bounds__(kNormThreads) mtrt_layernorm_##XN##_any(                        \
      const XT::storage* x, const XT::storage* gamma, const XT::storage* beta, XT::storage* y, int64_t rows,  \
      int64_t d, float eps) { layernorm_any<XT>(x, gamma, beta, y, rows, d, eps); }                           \
  extern "C" __global__ void __launch_bounds__(kNormThreads) mtrt_softmax_##XN##_any(                          \
      const XT::storage* x, XT::storage* y, int64_t rows, int64_t d) { softmax_any<XT>(x, y, rows, d); }

// One workgroup per row: mtrt_layernorm_<t>_g<THREADS>v<NV>(x, gamma, beta, y, rows, d, eps), mtrt_softmax_<t>_g<THREADS>v<NV>(x, y, rows, d)
//   grid = rows, block = THREADS; d % E == 0, d / E <= THREADS * NV, operands 16-byte aligned.
// Ragged rows: mtrt_{layernorm,softmax}_<t>_u<THREADS>v<NV>, same arguments; any d >= 1 with d / E <= THREADS * NV,
//   operands aligned to their element; THREADS <= 64 (NV = 1 below 64): grid = ceil(rows / (256 / THREADS)), block = 256;
//   else grid = rows, block = THREADS.
#define MTRT_NORM_GROUP_KERNELS(XN, XT, NV, THREADS, TAG, RAGGED, BLOCK)                                       \
  extern "C" __global__ void __launch_bounds__(BLOCK) mtrt_layernorm_##XN##_##TAG##THREADS##v##NV(             \
      const XT::storage* x, const XT::storage* gamma, const XT::storage* beta, XT::storage* y, int64_t rows,  \
      int64_t d, float eps) { layernorm_group<XT, NV, THREADS, RAGGED>(x, gamma, beta, y, rows, d, eps); }    \
  extern "C" __global__ void __launch_bounds__(BLOCK) mtrt_softmax_##XN##_##TAG##THREADS##v##NV(               \
      const XT::storage* x, XT::storage* y, int64_t rows, int64_t d) { softmax_group<XT, NV, THREADS, RAGGED>(x, y, rows, d); }
#define MTRT_NORM_GROUPS_FOR_TYPE(XN, XT)                                                                      \
  MTRT_NORM_GROUP_KERNELS(XN, XT, 8, 256, g, false, 256) MTRT_NORM_GROUP_KERNELS(XN, XT, 16, 256, g, false, 256)      \
  MTRT_NORM_GROUP_KERNELS(XN, XT, 8, 1024, g, false, 1024) MTRT_NORM_GROUP_KERNELS(XN, XT, 16, 1024, g, false, 1024)  \
  MTRT_NORM_GROUP_KERNELS(XN, XT, 1, 8, u, true, 256) MTRT_NORM_GROUP_KERNELS(XN, XT, 1, 16, u, true, 256)            \
  MTRT_NORM_GROUP_KERNELS(XN, XT, 1, 32, u, true, 256)                                                                \
  MTRT_NORM_GROUP_KERNELS(XN, XT, 1, 64, u, true, 256) MTRT_NORM_GROUP_KERNELS(XN, XT, 2, 64, u, true, 256)           \
  MTRT_NORM_GROUP_KERNELS(XN, XT, 4, 64, u, true, 256) MTRT_NORM_GROUP_KERNELS(XN, XT, 8, 64, u, true, 256)           \
  MTRT_NORM_GROUP_KERNELS(XN, XT, 16, 64, u, true, 256)                                                               \
  MTRT_NORM_GROUP_KERNELS(XN, XT, 8, 256, u, true, 256) MTRT_NORM_GROUP_KERNELS(XN, XT, 16, 256, u, true, 256)        \
  MTRT_NORM_GROUP_KERNELS(XN, XT, 8, 1024, u, true, 1024) MTRT_NORM_GROUP_KERNELS(XN, XT, 16, 1024, u, true, 1024)

MTRT_NORM_FOR_TYPE(f32, F32)
MTRT_NORM_FOR_TYPE(f16, F16)
MTRT_NORM_FOR_TYPE(bf16, BF16)
MTRT_NORM_GROUPS_FOR_TYPE(f32, F32)
MTRT_NORM_GROUPS_FOR_TYPE(f16, F16)
MTRT_NORM_GROUPS_FOR_TYPE(bf16, BF16)
