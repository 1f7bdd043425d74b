// Quantize / dequantize clusters for gfx950.
//
// Semantics (what each lane computes per element), following the reference's
// canonical StableHLO forms
//   quantize   : q = convert(clamp(lo, [round_nearest_even](f32(x) / scale), hi))
//                mlir-tensorrt/compiler/lib/Dialect/StablehloExt/Transforms/StablehloRaiseQDQ.cpp:233-265
//                mlir-tensorrt/tensorrt/include/mlir-tensorrt-dialect/TensorRT/IR/TensorRTOps.td:3133-3194
//   dequantize : y = narrow(f32(q) * scale)
//                StablehloRaiseQDQ.cpp:407-418 ; TensorRTOps.td:3408-3445
// with lo/hi = -128/127 (i8), -448/448 (f8E4M3FN), -8/7 (i4).  The quotient is always
// the correctly rounded IEEE f32 quotient - quantized codes must be bit-identical to
// the host lowering - computed either by the divide itself or, where many elements
// share one scale, by ExactDivisor below.
//
// Scale addressing (the data tensor is viewed as row-major [d0, d1]):
//   uniform : scale[0]                       per-tensor
//   row     : scale[row % nscale]            per-channel on a non-last axis, blocks along the last axis
//   col     : scale[(row / block) * d1 + c]  per-channel on the last axis (block = d0), blocks along axis 0
//
// Kernel arguments follow the reference's device ABI for generated kernels
// (mlir-tensorrt/kernel/lib/Kernel/Transforms/ExpandMemRefArgs.cpp:65-120): one
// bare pointer per buffer, then dynamic sizes as 64-bit integers, then scalars by
// value.
//
// Data movement.  The unit is a GROUP: the G consecutive elements that fill one
// 128-bit vector of the float operand (G = 4 for f32, 8 for f16/bf16).  In every
// memory instruction lane l of a wave touches group (base + l), so one instruction
// of a wave covers 64 consecutive groups: 1 KiB of the float operand and 256 or
// 512 contiguous bytes of codes, all whole cache lines.  A lane carries J groups
// per trip (16 elements), all loads issued before the first use.  The "_any"
// variants take any shape and alignment, one element per lane.
#include "common.hpp"

using namespace mtrt_dev;

namespace qdq_cluster {

// ---- float operand: one 128-bit vector <-> G floats ----------------------------
template <typename X> struct FloatGroup;
template <> struct FloatGroup<F32> {
  static constexpr int G = 4;
  static __device__ __forceinline__ u32x4 load(const float* p) { return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)); }
  static __device__ __forceinline__ void unpack(u32x4 t, float (&v)[4]) {
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] = bits_to_f32(t[k]);
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[4]) {
    u32x4 t = {f32_to_bits(v[0]), f32_to_bits(v[1]), f32_to_bits(v[2]), f32_to_bits(v[3])};
    __builtin_nontemporal_store(t, reinterpret_cast<u32x4*>(p));
  }
};
template <> struct FloatGroup<BF16> {
  static constexpr int G = 8;
  static __device__ __forceinline__ u32x4 load(const uint16_t* p) { return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)); }
  static __device__ __forceinline__ void unpack(u32x4 t, float (&v)[8]) {
#pragma unroll
    for (int k = 0; k < 4; ++k) { v[2 * k] = bits_to_f32(t[k] << 16); v[2 * k + 1] = bits_to_f32(t[k] & 0xFFFF0000u); }
  }
  static __device__ __forceinline__ void store(uint16_t* p, const float (&v)[8]) {
    u32x4 t;
#pragma unroll
    for (int k = 0; k < 4; ++k) t[k] = f32_to_bf16_bits(v[2 * k]) | (f32_to_bf16_bits(v[2 * k + 1]) << 16);
    __builtin_nontemporal_store(t, reinterpret_cast<u32x4*>(p));
  }
};
template <> struct FloatGroup<F16> {
  static constexpr int G = 8;
  static __device__ __forceinline__ u32x4 load(const uint16_t* p) { return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)); }
  static __device__ __forceinline__ void unpack(u32x4 t, float (&v)[8]) {
#pragma unroll
    for (int k = 0; k < 4; ++k) { v[2 * k] = f16_bits_to_f32(t[k] & 0xFFFFu); v[2 * k + 1] = f16_bits_to_f32(t[k] >> 16); }
  }
  static __device__ __forceinline__ void store(uint16_t* p, const float (&v)[8]) {
    u32x4 t;
#pragma unroll
    for (int k = 0; k < 4; ++k) t[k] = f32_to_f16_bits(v[2 * k]) | (f32_to_f16_bits(v[2 * k + 1]) << 16);
    __builtin_nontemporal_store(t, reinterpret_cast<u32x4*>(p));
  }
};

// ---- quantized codes ---------------------------------------------------------------
// enc(v): code of an already divided / rounded / clamped value.  dec(code): f32 value.
// A group of G codes travels as G/4 (bytes) or G/8 (nibbles) 32-bit words; the
// 4-nibble group of an f32 operand is a single 16-bit access.
template <typename Q> struct Codes;

template <> struct Codes<I8> {
  static constexpr float kLo = -128.0f, kHi = 127.0f;
  static constexpr bool kAlwaysRound = true;
  static __device__ __forceinline__ uint32_t enc(float v, int) { return uint32_t(int(v)) & 0xFFu; }
  static __device__ __forceinline__ float dec(uint32_t c) { return float(int(c << 24) >> 24); }
};
template <> struct Codes<F8> {
  static constexpr float kLo = -448.0f, kHi = 448.0f;
  static constexpr bool kAlwaysRound = false;
  static __device__ __forceinline__ uint32_t enc(float v, int flags) {
    if (flags & kFlagF8RefHost) return f32_to_f8_refhost(v);
    if (flags & kFlagF8ViaF16) v = f16_bits_to_f32(f32_to_f16_bits(v));
    return f32x2_to_f8_ieee(v, 0.0f) & 0xFFu;
  }
  static __device__ __forceinline__ float dec(uint32_t c) { return f8_to_f32<0>(c); }
};
// int4, one element per byte in the low nibble, upper nibble zero (host storage:
// DataTypes.cpp:494-519 keeps `bits_ & 0xF`).
template <> struct Codes<I4> {
  static constexpr float kLo = -8.0f, kHi = 7.0f;
  static constexpr bool kAlwaysRound = true;
  static __device__ __forceinline__ uint32_t enc(float v, int) { return uint32_t(int(v)) & 0xFu; }
  static __device__ __forceinline__ float dec(uint32_t c) { return float(int(c << 28) >> 28); }
};
// int4 packed two per byte over the flattened array, element 2i in the low nibble
// (mlir-tensorrt/tensorrt/lib/Target/TensorRTEncodingOpInterface/NetworkEncoder.cpp:552-595).
template <> struct Codes<I4P> {
  static constexpr float kLo = -8.0f, kHi = 7.0f;
  static constexpr bool kAlwaysRound = true;
  static __device__ __forceinline__ uint32_t enc(float v, int) { return uint32_t(int(v)) & 0xFu; }
  static __device__ __forceinline__ float dec(uint32_t c) { return float(int(c << 28) >> 28); }
};

// f4E2M1FN packed two per byte (element 2i in the low nibble).  The value goes through f16 first,
// the only f4 truncation the reference defines (RNE, saturation:
// mlir-tensorrt/executor/lib/Passes/ExpandOps.cpp:471-694); callers clamp to [-6, 6], so no NaN or
// infinity reaches the hardware conversion.
typedef _Float16 qdq_h2 __attribute__((ext_vector_type(2)));
typedef float qdq_f2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t f32x2_to_f4x2(float a, float b) {
  union { uint32_t u; qdq_h2 h; } c;
  c.u = f32_to_f16_bits(a) | (f32_to_f16_bits(b) << 16);
  return __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(0u, c.h, 1.0f, 0) & 0xFFu;
}
template <> struct Codes<F4P> {
  static constexpr float kLo = -6.0f, kHi = 6.0f;
  static constexpr bool kAlwaysRound = false;
  static __device__ __forceinline__ uint32_t enc(float v, int) { return f32x2_to_f4x2(v, 0.0f) & 0xFu; }
  static __device__ __forceinline__ float dec(uint32_t c) { return __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(c & 0xFu, 1.0f, 0)[0]; }
};

// Four byte-wide codes <-> one 32-bit word.  The f8 IEEE path converts pairs in
// hardware; everything else goes through enc/dec.
template <typename Q>
__device__ __forceinline__ uint32_t pack4(const float* v, int flags) {
  return Codes<Q>::enc(v[0], flags) | (Codes<Q>::enc(v[1], flags) << 8) | (Codes<Q>::enc(v[2], flags) << 16) |
         (Codes<Q>::enc(v[3], flags) << 24);
}
template <>
__device__ __forceinline__ uint32_t pack4<F8>(const float* v, int flags) {
  if (flags & kFlagF8RefHost) {
    // The host class (f32_to_f8_refhost) equals the hardware's round-to-nearest-even except that every result with
    // the top exponent (256 .. 448) becomes 448, and that it rounds differently below the normal range
    // (2^-10 <= |v| < 2^-6; smaller values are zero both ways).  So: the hardware conversion, the top exponent
    // fixed up on the four bytes at once, and the software form only for the elements, and in the waves, where a lane
    // holds such a small value (with scales derived from amax about one value in 10^4).
    int hw = __builtin_amdgcn_cvt_pk_fp8_f32(v[0], v[1], 0, false);
    hw = __builtin_amdgcn_cvt_pk_fp8_f32(v[2], v[3], hw, true);
    uint32_t codes = uint32_t(hw);
    const uint32_t top = (((codes & 0x7F7F7F7Fu) + 0x08080808u) >> 7) & 0x01010101u;   // magnitude >= 0x78, per byte
    codes = (codes | (top * 0x7Eu)) & ~top;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const bool small = ((f32_to_bits(v[k]) & 0x7FFFFFFFu) - 0x3A800000u) < 0x02000000u;
      if (__builtin_amdgcn_ballot_w64(small)) {
        if (small) codes = (codes & ~(0xFFu << (8 * k))) | (f32_to_f8_refhost(v[k]) << (8 * k));
      }
    }
    return codes;
  }
  // The reference's generated GPU code never converts f32 to f8 directly: it truncates to f16 first and
  // converts that (mlir-tensorrt/kernel/lib/Kernel/Transforms/NormalizeQuantizedConversions.cpp:38-118,
  // cvt.rn.satfinite.e4m3x2.f16x2 in LowerToNVVM.cpp:281-339).  Both steps round to nearest even, so a value
  // within half an f16 ulp of an f8 midpoint first lands ON the midpoint and then goes to the even code.
  // Widening f16 to f32 is exact, so the second step can use the f32 conversion instruction.
  float t[4] = {v[0], v[1], v[2], v[3]};
  if (flags & kFlagF8ViaF16) {
#pragma unroll
    for (int k = 0; k < 4; ++k) t[k] = f16_bits_to_f32(f32_to_f16_bits(t[k]));
  }
  int w = __builtin_amdgcn_cvt_pk_fp8_f32(t[0], t[1], 0, false);
  return uint32_t(__builtin_amdgcn_cvt_pk_fp8_f32(t[2], t[3], w, true));
}
template <typename Q>
__device__ __forceinline__ void unpack4(uint32_t w, float* v) {
#pragma unroll
  for (int k = 0; k < 4; ++k) v[k] = Codes<Q>::dec((w >> (8 * k)) & 0xFFu);
}
template <>
__device__ __forceinline__ void unpack4<F8>(uint32_t w, float* v) {
  v[0] = f8_to_f32<0>(w); v[1] = f8_to_f32<1>(w); v[2] = f8_to_f32<2>(w); v[3] = f8_to_f32<3>(w);
}

// G codes of one group, at element offset `e` (a multiple of G) of the code array.
// store() leaves f32(code) in v[]: the value a following dequantize multiplies by
// the scale (this also turns the -0.0 a rounding can produce into the +0.0 that
// reading the integer code back gives).
template <typename Q, int G> struct CodeGroup {
  static constexpr int kWords = G / 4;
  static __device__ __forceinline__ void store(typename Q::storage* base, int64_t e, float (&v)[G], int flags) {
    uint32_t w[kWords];
#pragma unroll
    for (int i = 0; i < kWords; ++i) { w[i] = pack4<Q>(&v[4 * i], flags); unpack4<Q>(w[i], &v[4 * i]); }
    if (kWords == 1) {
      __builtin_nontemporal_store(w[0], reinterpret_cast<uint32_t*>(base + e));
    } else {
      u32x2 t = {w[0], w[kWords - 1]};
      __builtin_nontemporal_store(t, reinterpret_cast<u32x2*>(base + e));
    }
  }
  static __device__ __forceinline__ void load_raw(const typename Q::storage* base, int64_t e, uint32_t (&w)[2]) {
    if (kWords == 1) {
      w[0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(base + e));
    } else {
      const u32x2 t = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(base + e));
      w[0] = t.x; w[1] = t.y;
    }
  }
  static __device__ __forceinline__ void decode(const uint32_t (&w)[2], float (&v)[G]) {
#pragma unroll
    for (int i = 0; i < kWords; ++i) unpack4<Q>(w[i], &v[4 * i]);
  }
};
template <int G> struct CodeGroup<I4P, G> {
  static __device__ __forceinline__ void store(uint8_t* base, int64_t e, float (&v)[G], int) {
    uint32_t w = 0;
#pragma unroll
    for (int k = 0; k < G; ++k) {
      const int c = int(v[k]);
      v[k] = float(c);
      w |= (uint32_t(c) & 0xFu) << (4 * k);
    }
    if (G == 4) __builtin_nontemporal_store(uint16_t(w), reinterpret_cast<uint16_t*>(base + (e >> 1)));
    else __builtin_nontemporal_store(w, reinterpret_cast<uint32_t*>(base + (e >> 1)));
  }
  static __device__ __forceinline__ void load_raw(const uint8_t* base, int64_t e, uint32_t (&w)[2]) {
    if (G == 4) w[0] = __builtin_nontemporal_load(reinterpret_cast<const uint16_t*>(base + (e >> 1)));
    else w[0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(base + (e >> 1)));
  }
  static __device__ __forceinline__ void decode(const uint32_t (&w)[2], float (&v)[G]) {
#pragma unroll
    for (int k = 0; k < G; ++k) v[k] = float(int(w[0] << (28 - 4 * k)) >> 28);
  }
};

template <int G> struct CodeGroup<F4P, G> {
  static __device__ __forceinline__ void store(uint8_t* base, int64_t e, float (&v)[G], int) {
    uint32_t w = 0;
#pragma unroll
    for (int k = 0; k < G; k += 2) w |= f32x2_to_f4x2(v[k], v[k + 1]) << (4 * k);
    const uint32_t keep[2] = {w, 0};
    decode(keep, v);
    if (G == 4) __builtin_nontemporal_store(uint16_t(w), reinterpret_cast<uint16_t*>(base + (e >> 1)));
    else __builtin_nontemporal_store(w, reinterpret_cast<uint32_t*>(base + (e >> 1)));
  }
  static __device__ __forceinline__ void load_raw(const uint8_t* base, int64_t e, uint32_t (&w)[2]) {
    if (G == 4) w[0] = __builtin_nontemporal_load(reinterpret_cast<const uint16_t*>(base + (e >> 1)));
    else w[0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(base + (e >> 1)));
  }
  static __device__ __forceinline__ void decode(const uint32_t (&w)[2], float (&v)[G]) {
    qdq_f2 p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[0], 1.0f, 0);
    v[0] = p[0]; v[1] = p[1];
    p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[0], 1.0f, 1);
    v[2] = p[0]; v[3] = p[1];
    if (G == 8) {
      p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[0], 1.0f, 2);
      v[4 % G] = p[0]; v[5 % G] = p[1];
      p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[0], 1.0f, 3);
      v[6 % G] = p[0]; v[7 % G] = p[1];
    }
  }
};

// round (where the target asks for it) and clamp an exact quotient
template <typename Q>
__device__ __forceinline__ float finish_quotient(float v, int flags) {
  if (Codes<Q>::kAlwaysRound || (flags & kFlagRoundToInt))
    v = __builtin_rintf(v);                          // v_rndne_f32: exact round-half-even
  return fmaxf(fminf(v, Codes<Q>::kHi), Codes<Q>::kLo);
}
template <typename Q>
__device__ __forceinline__ float quant_value(float x, float s, int flags) {
  return finish_quotient<Q>(x / s, flags);           // IEEE divide, bit-exact with the host
}

// Correctly rounded x / s for MANY x and ONE s, in 8 instructions instead of the 13
// of the full IEEE divide expansion.  With r = RN(1/s) (one IEEE divide per lane):
//     q0 = RN(x r);  q1 = RN(q0 + RN(x - q0 s) r);  q2 = RN(q1 + RN(x - q1 s) r)
// q1 is within a hair of x/s, hence a faithful rounding, and the remainder of a
// faithful quotient is exact in an FMA; Markstein's theorem (a faithful quotient
// corrected once with the correctly rounded reciprocal is the correctly rounded
// quotient) then gives q2 = RN(x/s).  The theorem needs no overflow or underflow in
// the intermediates, which the guards provide: |s| must lie in [2^-60, 2^60] (else
// the lane-uniform slow path divides), and x is first clamped to +-1024|s|, beyond
// which every target saturates anyway; min/max drop a NaN x to the positive bound,
// which saturates high exactly as the NaN quotient does in the clamp of the plain
// path.  Quotients too small for an exact remainder (|x| < 2^-100) are far below
// half the least code of every target and produce the same signed zero either way.
struct ExactDivisor {
  float s, r, bound;
  bool fast;
  ExactDivisor() = default;
  __device__ __forceinline__ explicit ExactDivisor(float scale) : s(scale) {
    const uint32_t e = (f32_to_bits(scale) >> 23) & 0xFFu;
    fast = e >= 127u - 60u && e <= 127u + 60u;
    r = 1.0f / scale;
    bound = 1024.0f * fabsf(scale);
  }
  __device__ __forceinline__ float divide(float x) const {
    if (!fast) return x / s;
    const float xc = fmaxf(fminf(x, bound), -bound);
    const float q0 = xc * r;
    float q = __builtin_fmaf(__builtin_fmaf(-q0, s, xc), r, q0);
    q = __builtin_fmaf(__builtin_fmaf(-q, s, xc), r, q);
    // A zero quotient must keep the sign the divide gives it (-0.0 / s = -0.0, and an
    // f8 code carries that sign); the corrections add +0 and would lose it.  q0 always
    // has the sign of the true quotient.
    return __builtin_copysignf(q, q0);
  }
  // The group form of the fast path: quotient, rounding (ROUND) and the target's clamp for G values at once, for
  // callers that have checked `fast` for the whole wave.  Same values as finish_quotient(divide(x)); the sign of
  // zero is put back after the clamp (a clamp keeps it), so that the clamp's operands are results of arithmetic
  // and need no quieting first.
  template <typename Q, bool ROUND>
  __device__ __forceinline__ float quantize_fast1(float x) const {
    const float xc = fmaxf(fminf(x, bound), -bound);
    const float q0 = xc * r;
    float q = __builtin_fmaf(__builtin_fmaf(-q0, s, xc), r, q0);
    q = __builtin_fmaf(__builtin_fmaf(-q, s, xc), r, q);
    if (ROUND) q = __builtin_rintf(q);
    q = fmaxf(fminf(q, Codes<Q>::kHi), Codes<Q>::kLo);
    return __builtin_copysignf(q, q0);
  }
  template <typename Q, bool ROUND, int G>
  __device__ __forceinline__ void quantize_fast(float (&v)[G]) const {
#pragma unroll
    for (int k = 0; k < G; ++k) v[k] = quantize_fast1<Q, ROUND>(v[k]);
  }
};

// G values that share one scale -> their clamped (and, where asked for, rounded) quotients.  Both choices, the
// short division for every lane of the wave or not, and rounding or not, are branches of the whole wave around
// loops over the group, not selects per element.
template <typename Q, int G>
__device__ __forceinline__ void quantize_group(const ExactDivisor& dv, float (&v)[G], int flags) {
  const bool round = Codes<Q>::kAlwaysRound || (flags & kFlagRoundToInt);
  if (__builtin_amdgcn_ballot_w64(!dv.fast) == 0) {
    if (round) dv.template quantize_fast<Q, true>(v);
    else dv.template quantize_fast<Q, false>(v);
  } else {
#pragma unroll
    for (int k = 0; k < G; ++k) v[k] = finish_quotient<Q>(dv.divide(v[k]), flags);
  }
}

enum ScaleKind { kUniform = 0, kRow = 1, kCol = 2 };

// Column scales (per-channel on the last axis, blocks of nb rows): in the group loop below every group fetches its
// own G scales and divides by each once, so the scales cost as many bytes through the vector cache as the tensor
// and every element an IEEE divide.  Here a wave takes a STRIP of 64 groups of columns and walks kColChunkRows
// rows of one scale block down it: the lane's G scales are fetched, and their reciprocals formed, once per strip
// and chunk; every row of the chunk is one contiguous KiB of the float operand per wave, as before.
// Host guarantees as for qdq_groups<kCol>: d1 % G == 0, n / G < 2^32, operands aligned for group accesses,
// the scales 16-byte aligned.
constexpr int kColChunkRows = 32;

template <typename X, typename Q, int MODE>
__device__ __forceinline__ void qdq_col_strips(const typename X::storage* __restrict__ x, typename Q::storage* __restrict__ q,
                                               typename X::storage* __restrict__ y, const float* __restrict__ scale,
                                               int64_t n, int64_t d1, int64_t nb, int flags) {
  using FG = FloatGroup<X>;
  constexpr int G = FG::G;
  constexpr int U = 4;                               // rows in flight per lane
  using CG = CodeGroup<Q, G>;
  const uint32_t groups_per_row = uint32_t(d1 / G), strips = (groups_per_row + kWave - 1) / kWave;
  const int64_t d0 = n / d1, nblocks = d0 / nb;
  const uint32_t chunks = uint32_t((nb + kColChunkRows - 1) / kColChunkRows);
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = (int64_t(blockIdx.x) * blockDim.x + threadIdx.x) / kWave;
  const int64_t nwaves = int64_t(gridDim.x) * blockDim.x / kWave;
  const int64_t items = nblocks * chunks * strips;
  const bool round = Codes<Q>::kAlwaysRound || (flags & kFlagRoundToInt);

  for (int64_t item = wave; item < items; item += nwaves) {
    const uint32_t strip = uint32_t(item % strips);
    const int64_t rest = item / strips;
    const uint32_t chunk = uint32_t(rest % chunks);
    const int64_t b = rest / chunks;
    const uint32_t cg = strip * kWave + lane;
    const bool live = cg < groups_per_row;
    const int64_t c0 = int64_t(live ? cg : groups_per_row - 1) * G;     // idle lanes repeat the last group, store nothing
    float sc[G];
    const f32x4* sp = reinterpret_cast<const f32x4*>(scale + b * d1 + c0);
#pragma unroll
    for (int k = 0; k < G / 4; ++k) {
      const f32x4 t = sp[k];
      sc[4 * k] = t.x; sc[4 * k + 1] = t.y; sc[4 * k + 2] = t.z; sc[4 * k + 3] = t.w;
    }
    const int64_t r0 = b * nb + int64_t(chunk) * kColChunkRows;
    const int64_t r1 = r0 + kColChunkRows < (b + 1) * nb ? r0 + kColChunkRows : (b + 1) * nb;
    ExactDivisor dv[G];
    bool fast = true;
#pragma unroll
    for (int k = 0; k < G; ++k) {
      if (MODE != 1) dv[k] = ExactDivisor(sc[k]);
      fast = fast && (MODE == 1 || dv[k].fast);
    }
    const bool all_fast = MODE == 1 || __builtin_amdgcn_ballot_w64(!fast) == 0;

    for (int64_t r = r0; r < r1; r += U) {
      u32x4 xin[U];
      uint32_t qin[U][2];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t e = (r + u < r1 ? r + u : r1 - 1) * d1 + c0;
        if (MODE == 1) CG::load_raw(q, e, qin[u]);
        else xin[u] = FG::load(x + e);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t e = (r + u) * d1 + c0;
        const bool store = live && r + u < r1;
        float v[G];
        if (MODE == 1) {
          CG::decode(qin[u], v);
        } else {
          FG::unpack(xin[u], v);
          if (all_fast) {
            if (round) {
#pragma unroll
              for (int k = 0; k < G; ++k) v[k] = dv[k].template quantize_fast1<Q, true>(v[k]);
            } else {
#pragma unroll
              for (int k = 0; k < G; ++k) v[k] = dv[k].template quantize_fast1<Q, false>(v[k]);
            }
          } else {
#pragma unroll
            for (int k = 0; k < G; ++k) v[k] = quant_value<Q>(v[k], sc[k], flags);
          }
          if (store) CG::store(q, e, v, flags);       // leaves f32(code) in v
        }
        if (MODE != 0 && store) {
#pragma unroll
          for (int k = 0; k < G; ++k) v[k] = v[k] * sc[k];
          FG::store(y + e, v);
        }
      }
    }
  }
}

// MODE: 0 = quantize (write q), 1 = dequantize (read q, write y),
//       2 = fused quantize->dequantize (read x, write q and y)
// Host guarantees: n < 2^35; for row/col scales d1 % G == 0 (a group never
// straddles rows); operands aligned for their group accesses.
template <typename X, typename Q, int KIND, int MODE>
__device__ __forceinline__ void qdq_groups(const typename X::storage* __restrict__ x, typename Q::storage* __restrict__ q,
                                           typename X::storage* __restrict__ y, const float* __restrict__ scale,
                                           int64_t n, int64_t d1, int64_t nb, int flags) {
  using FG = FloatGroup<X>;
  constexpr int G = FG::G;
  constexpr int J = kTile / G;                       // groups per lane per trip
  constexpr int SN = KIND == kCol ? G : 1;           // scale values a lane needs per group
  using CG = CodeGroup<Q, G>;
  const int64_t ngroups = n / G;
  const uint32_t groups_per_row = KIND == kUniform ? 1u : uint32_t(d1 / G);
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = (int64_t(blockIdx.x) * blockDim.x + threadIdx.x) / kWave;
  const int64_t nwaves = int64_t(gridDim.x) * blockDim.x / kWave;
  const float s_uniform = KIND == kUniform ? scale[0] : 0.0f;

  for (int64_t base = wave * (kWave * J); base < ngroups; base += nwaves * (kWave * J)) {
    float v[J][G];
    float s[J][SN];
    bool live[J];
    u32x4 xin[J];
    uint32_t qin[J][2];
    // all loads of the trip first
#pragma unroll
    for (int j = 0; j < J; ++j) {
      const int64_t g = base + j * kWave + lane;
      live[j] = g < ngroups;
      if (!live[j]) continue;
      if (MODE == 1) CG::load_raw(q, g * G, qin[j]);
      else xin[j] = FG::load(x + g * G);
      if (KIND == kUniform) {
        s[j][0] = s_uniform;
      } else {
        // group, row and scale indices are below 2^32 for anything that fits in HBM
        const uint32_t row = uint32_t(g) / groups_per_row;
        if (KIND == kRow) {
          s[j][0] = scale[row % uint32_t(nb)];
        } else {
          const int64_t c0 = int64_t(uint32_t(g) - row * groups_per_row) * G;
          const f32x4* sp = reinterpret_cast<const f32x4*>(scale + int64_t(row / uint32_t(nb)) * d1 + c0);
#pragma unroll
          for (int k = 0; k < SN / 4; ++k) {
            const f32x4 t = sp[k];
            s[j][(4 * k + 0) % SN] = t.x; s[j][(4 * k + 1) % SN] = t.y;
            s[j][(4 * k + 2) % SN] = t.z; s[j][(4 * k + 3) % SN] = t.w;
          }
        }
      }
    }
#pragma unroll
    for (int j = 0; j < J; ++j) {
      if (!live[j]) continue;
      const int64_t e = (base + j * kWave + lane) * G;
      if (MODE == 1) {
        CG::decode(qin[j], v[j]);
      } else {
        FG::unpack(xin[j], v[j]);
        if (KIND == kCol) {
#pragma unroll
          for (int k = 0; k < G; ++k) v[j][k] = quant_value<Q>(v[j][k], s[j][k % SN], flags);
        } else {
          // one scale for the whole group: exact division through its reciprocal
          const ExactDivisor dv(s[j][0]);
          quantize_group<Q>(dv, v[j], flags);
        }
        CG::store(q, e, v[j], flags);
      }
      if (MODE != 0) {
#pragma unroll
        for (int k = 0; k < G; ++k) v[j][k] = v[j][k] * s[j][k % SN];
        FG::store(y + e, v[j]);
      }
    }
  }

  // Remainder (< G elements) of a per-tensor array, one lane each; row- and
  // column-scaled launches have n % G == 0 by construction.  Packed nibbles: the
  // lane of the even element writes the whole byte.
  if (KIND == kUniform && blockIdx.x == 0 && threadIdx.x < G) {
    const int64_t e = ngroups * G + threadIdx.x;
    if (e < n) {
      if (Q::kBits == 4) {
        if ((e & 1) == 0) {
          const bool has1 = e + 1 < n;
          float v0, v1 = 0.0f;
          if (MODE == 1) {
            const uint32_t byte = uint32_t(uint8_t(q[e >> 1]));
            v0 = Codes<Q>::dec(byte & 0xFu);
            v1 = Codes<Q>::dec(byte >> 4);
          } else {
            v0 = quant_value<Q>(Tile<X>::load1(x + e), s_uniform, flags);
            if (has1) v1 = quant_value<Q>(Tile<X>::load1(x + e + 1), s_uniform, flags);
            const uint32_t c0 = Codes<Q>::enc(v0, flags), c1 = Codes<Q>::enc(v1, flags);
            q[e >> 1] = typename Q::storage(c0 | (c1 << 4));
            v0 = Codes<Q>::dec(c0); v1 = Codes<Q>::dec(c1);
          }
          if (MODE != 0) {
            Tile<X>::store1(y + e, v0 * s_uniform);
            if (has1) Tile<X>::store1(y + e + 1, v1 * s_uniform);
          }
        }
      } else {
        float v;
        if (MODE == 1) {
          v = Codes<Q>::dec(uint32_t(uint8_t(q[e])));
        } else {
          v = quant_value<Q>(Tile<X>::load1(x + e), s_uniform, flags);
          const uint32_t c = Codes<Q>::enc(v, flags);
          q[e] = typename Q::storage(c);
          v = Codes<Q>::dec(c);
        }
        if (MODE != 0) Tile<X>::store1(y + e, v * s_uniform);
      }
    }
  }
}

// Row and column scales on rows that are not whole groups (d1 % G != 0) or on operands that are not aligned for group
// accesses: the element-per-lane kernel below moves one or two bytes per lane and instruction and runs at a sixth of
// the memory rate.  Here a wave takes 64 consecutive groups of ONE row at a time, with 128-bit accesses at element
// alignment (the hardware splits those that straddle a cache line) and the codes as unaligned 4- or 8-byte stores;
// the d1 % G elements behind a row's last whole group go one each to the first lanes.  A group never straddles rows,
// so a row scale is uniform per group (short exact division, as in qdq_groups) and column scales are G consecutive
// floats.  Codes one per byte (i8, f8, i4); packed nibbles stay with the kernel below (a byte can straddle rows).
typedef u32x4 u32x4_unaligned __attribute__((aligned(2)));
typedef f32x4 f32x4_unaligned __attribute__((aligned(4)));
typedef uint32_t u32_unaligned __attribute__((aligned(1)));

template <typename X, typename Q, int KIND, int MODE>
__device__ __forceinline__ void qdq_rows_ragged(const typename X::storage* __restrict__ x, typename Q::storage* __restrict__ q,
                                                typename X::storage* __restrict__ y, const float* __restrict__ scale,
                                                int64_t n, int64_t d1, int64_t nb, int64_t fpitch, int64_t qpitch, int flags) {
  using FG = FloatGroup<X>;
  constexpr int G = FG::G;
  const int64_t d0 = n / d1, nvec = d1 / G;
  const int tail = int(d1 - nvec * G);
  const int64_t chunks = nvec > 0 ? (nvec + kWave - 1) / kWave : 1;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = (int64_t(blockIdx.x) * blockDim.x + threadIdx.x) / kWave;
  const int64_t nwaves = int64_t(gridDim.x) * blockDim.x / kWave;
  const int64_t items = d0 * chunks;
  for (int64_t item = wave; item < items; item += nwaves) {
    const int64_t row = item / chunks, c = item - row * chunks;
    const int64_t v = c * kWave + lane;
    const int64_t fe0 = row * fpitch + v * G, qe0 = row * qpitch + v * G;   // row pitches in elements: d1 unless the operand is a view
    const float* srow = KIND == kRow ? scale + row % nb : scale + (row / nb) * d1;
    if (v < nvec) {
      float f[G], sc[G];
      if (KIND == kRow) {
        const float s = srow[0];
#pragma unroll
        for (int k = 0; k < G; ++k) sc[k] = s;
      } else {
#pragma unroll
        for (int k = 0; k < G / 4; ++k) {
          const f32x4 t = *reinterpret_cast<const f32x4_unaligned*>(srow + v * G + 4 * k);
          sc[4 * k] = t.x; sc[4 * k + 1] = t.y; sc[4 * k + 2] = t.z; sc[4 * k + 3] = t.w;
        }
      }
      uint32_t w[G / 4];
      if (MODE == 1) {
#pragma unroll
        for (int i = 0; i < G / 4; ++i) {
          w[i] = *reinterpret_cast<const u32_unaligned*>(q + qe0 + 4 * i);
          unpack4<Q>(w[i], &f[4 * i]);
        }
      } else {
        const u32x4 t = *reinterpret_cast<const u32x4_unaligned*>(x + fe0);
        FG::unpack(t, f);
        if (KIND == kRow) {
          const ExactDivisor dv(sc[0]);
          quantize_group<Q>(dv, f, flags);
        } else {
#pragma unroll
          for (int k = 0; k < G; ++k) f[k] = quant_value<Q>(f[k], sc[k], flags);
        }
#pragma unroll
        for (int i = 0; i < G / 4; ++i) {
          w[i] = pack4<Q>(&f[4 * i], flags);
          unpack4<Q>(w[i], &f[4 * i]);                 // f32(code): what a following dequantize multiplies
          *reinterpret_cast<u32_unaligned*>(q + qe0 + 4 * i) = w[i];
        }
      }
      if (MODE != 0) {
#pragma unroll
        for (int k = 0; k < G; ++k) f[k] = f[k] * sc[k];
        u32x4 t;
        if (G == 4) {
          t = (u32x4){f32_to_bits(f[0]), f32_to_bits(f[1]), f32_to_bits(f[2]), f32_to_bits(f[3])};
          *reinterpret_cast<u32x4_unaligned*>(y + fe0) = t;
        } else {
          // 16-bit outputs: narrowed one by one through the element form, then stored as one vector
          typename X::storage h[8];
#pragma unroll
          for (int k = 0; k < 8; ++k) Tile<X>::store1(&h[k % G], f[k % G]);
#pragma unroll
          for (int k = 0; k < 4; ++k) t[k] = uint32_t(uint16_t(h[(2 * k) % G])) | (uint32_t(uint16_t(h[(2 * k + 1) % G])) << 16);
          *reinterpret_cast<u32x4_unaligned*>(y + fe0) = t;
        }
      }
    }
    if (c == chunks - 1 && lane < tail) {              // the row's last d1 % G elements, one per lane
      const int64_t col = nvec * G + lane, fe = row * fpitch + col, qe = row * qpitch + col;
      const float s = KIND == kRow ? srow[0] : srow[col];
      float fv;
      if (MODE == 1) {
        fv = Codes<Q>::dec(uint32_t(uint8_t(q[qe])));
      } else {
        fv = quant_value<Q>(Tile<X>::load1(x + fe), s, flags);
        const uint32_t code = Codes<Q>::enc(fv, flags);
        q[qe] = typename Q::storage(code);
        fv = Codes<Q>::dec(code);
      }
      if (MODE != 0) Tile<X>::store1(y + fe, fv * s);
    }
  }
}

// Any shape, any alignment: one element per lane (packed int4: one byte = two
// elements per lane), scale kind chosen at run time.
template <typename X, typename Q, int MODE>
__device__ __forceinline__ void qdq_any(const typename X::storage* __restrict__ x, typename Q::storage* __restrict__ q,
                                        typename X::storage* __restrict__ y, const float* __restrict__ scale,
                                        int64_t n, int64_t d1, int64_t nb, int kind, int flags) {
  constexpr int kPer = (Q::kBits == 4) ? 2 : 1;
  const int64_t units = (n + kPer - 1) / kPer;
  const int64_t stride = int64_t(gridDim.x) * blockDim.x;
  for (int64_t u = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; u < units; u += stride) {
    uint32_t byte = (Q::kBits == 4 && MODE == 1) ? uint32_t(uint8_t(q[u])) : 0u;
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
      const int64_t e = u * kPer + k;
      if (e >= n) continue;
      const int64_t row = e / d1;
      const float s = kind == kUniform ? scale[0]
                                       : (kind == kRow ? scale[row % nb] : scale[(row / nb) * d1 + (e - row * d1)]);
      float v;
      if (MODE == 1) {
        v = Q::kBits == 4 ? Codes<Q>::dec((byte >> (4 * k)) & 0xFu) : Codes<Q>::dec(uint32_t(uint8_t(q[e])));
      } else {
        v = quant_value<Q>(Tile<X>::load1(x + e), s, flags);
        const uint32_t c = Codes<Q>::enc(v, flags);
        if (Q::kBits == 4) byte |= c << (4 * k);
        else q[e] = typename Q::storage(c);
        v = Codes<Q>::dec(c);
      }
      if (MODE != 0) Tile<X>::store1(y + e, v * s);
    }
    if (Q::kBits == 4 && MODE != 1) q[u] = typename Q::storage(byte);
  }
}

}  // namespace qdq_cluster
using namespace qdq_cluster;

// ---- entry points -----------------------------------------------------------------
// Names: mtrt_{q,dq,qdq}_{uniform,row,col,any}_<float type>_<code type>
//   q   (x, q, scale, n, d1, nb, flags)        dq  (q, y, scale, n, d1, nb)
//   qdq (x, q, y, scale, n, d1, nb, flags)     *_any add `kind` after nb
#define MTRT_QDQ_KERNELS(XN, XT, QN, QT)                                                                          \
  extern "C" __global__ void __launch_bounds__(256) mtrt_q_uniform_##XN##_##QN(                                   \
      const XT::storage* x, QT::storage* q, const float* scale, int64_t n, int64_t d1, int64_t nb, int32_t flags) { \
    qdq_groups<XT, QT, kUniform, 0>(x, q, nullptr, scale, n, d1, nb, flags); }                                    \
  extern "C" __global__ void __launch_bounds__(256) mtrt_q_row_##XN##_##QN(                                       \
      const XT::storage* x, QT::storage* q, const float* scale, int64_t n, int64_t d1, int64_t nb, int32_t flags) { \
    qdq_groups<XT, QT, kRow, 0>(x, q, nullptr, scale, n, d1, nb, flags); }                                        \
  extern "C" __global__ void __launch_bounds__(256) mtrt_q_col_##XN##_##QN(                                       \
      const XT::storage* x, QT::storage* q, const float* scale, int64_t n, int64_t d1, int64_t nb, int32_t flags) { \
    qdq_col_strips<XT, QT, 0>(x, q, nullptr, scale, n, d1, nb, flags); }                                        \
  extern "C" __global__ void __launch_bounds__(256) mtrt_q_any_##XN##_##QN(                                       \
      const XT::storage* x, QT::storage* q, const float* scale, int64_t n, int64_t d1, int64_t nb, int32_t kind,  \
      int32_t flags) { qdq_any<XT, QT, 0>(x, q, nullptr, scale, n, d1, nb, kind, flags); }                        \
  extern "C" __global__ void __launch_bounds__(256) mtrt_dq_uniform_##XN##_##QN(                                  \
      const QT::storage* q, XT::storage* y, const float* scale, int64_t n, int64_t d1, int64_t nb) {              \
    qdq_groups<XT, QT, kUniform, 1>(nullptr, const_cast<QT::storage*>(q), y, scale, n, d1, nb, 0); }              \
  extern "C" __global__ void __launch_bounds__(256) mtrt_dq_row_##XN##_##QN(                                      \
      const QT::storage* q, XT::storage* y, const float* scale, int64_t n, int64_t d1, int64_t nb) {              \
    qdq_groups<XT, QT, kRow, 1>(nullptr, const_cast<QT::storage*>(q), y, scale, n, d1, nb, 0); }                  \
  extern "C" __global__ void __launch_bounds__(256) mtrt_dq_col_##XN##_##QN(                                      \
      const QT::storage* q, XT::storage* y, const float* scale, int64_t n, int64_t d1, int64_t nb) {              \
    qdq_col_strips<XT, QT, 1>(nullptr, const_cast<QT::storage*>(q), y, scale, n, d1, nb, 0); }                  \
  extern "C" __global__ void __launch_bounds__(256) mtrt_dq_any_##XN##_##QN(                                      \
      const QT::storage* q, XT::storage* y, const float* scale, int64_t n, int64_t d1, int64_t nb, int32_t kind) { \
    qdq_any<XT, QT, 1>(nullptr, const_cast<QT::storage*>(q), y, scale, n, d1, nb, kind, 0); }                     \
  extern "C" __global__ void __launch_bounds__(256) mtrt_qdq_uniform_##XN##_##QN(                                 \
      const XT::storage* x, QT::storage* q, XT::storage* y, const float* scale, int64_t n, int64_t d1, int64_t nb, \
      int32_t flags) { qdq_groups<XT, QT, kUniform, 2>(x, q, y, scale, n, d1, nb, flags); }                       \
  extern "C" __global__ void __launch_bounds__(256) mtrt_qdq_row_##XN##_##QN(                                     \
      const XT::storage* x, QT::storage* q, XT::storage* y, const float* scale, int64_t n, int64_t d1, int64_t nb, \
      int32_t flags) { qdq_groups<XT, QT, kRow, 2>(x, q, y, scale, n, d1, nb, flags); }                           \
  extern "C" __global__ void __launch_bounds__(256) mtrt_qdq_col_##XN##_##QN(                                     \
      const XT::storage* x, QT::storage* q, XT::storage* y, const float* scale, int64_t n, int64_t d1, int64_t nb, \
      int32_t flags) { qdq_col_strips<XT, QT, 2>(x, q, y, scale, n, d1, nb, flags); }                           \
  extern "C" __global__ void __launch_bounds__(256) mtrt_qdq_any_##XN##_##QN(                                     \
      const XT::storage* x, QT::storage* q, XT::storage* y, const float* scale, int64_t n, int64_t d1, int64_t nb, \
      int32_t kind, int32_t flags) { qdq_any<XT, QT, 2>(x, q, y, scale, n, d1, nb, kind, flags); }

#define MTRT_QDQ_FOR_FLOAT(XN, XT)    \
  MTRT_QDQ_KERNELS(XN, XT, i8, I8)    \
  MTRT_QDQ_KERNELS(XN, XT, f8, F8)    \
  MTRT_QDQ_KERNELS(XN, XT, i4, I4)    \
  MTRT_QDQ_KERNELS(XN, XT, i4p, I4P)   \
  MTRT_QDQ_KERNELS(XN, XT, f4p, F4P)

MTRT_QDQ_FOR_FLOAT(f32, F32)
MTRT_QDQ_FOR_FLOAT(f16, F16)
MTRT_QDQ_FOR_FLOAT(bf16, BF16)

// Ragged rows / unaligned operands with row or column scales: mtrt_{q,dq,qdq}_{rowu,colu}_<float type>_<code type>,
// arguments as the kernels above plus, behind nb, the row pitches in elements of the float operand(s) and of the codes
// (d1 for contiguous tensors; views with unit inner stride pass their row strides); grid-stride over (row, chunk of
// 64 groups), block = 256; codes i8, f8, i4.
#define MTRT_QDQ_RAGGED_KERNELS(XN, XT, QN, QT, KN, KIND)                                                          \
  extern "C" __global__ void __launch_bounds__(256) mtrt_q_##KN##_##XN##_##QN(                                     \
      const XT::storage* x, QT::storage* q, const float* scale, int64_t n, int64_t d1, int64_t nb, int64_t fpitch, \
      int64_t qpitch, int32_t flags) { qdq_rows_ragged<XT, QT, KIND, 0>(x, q, nullptr, scale, n, d1, nb, fpitch, qpitch, flags); } \
  extern "C" __global__ void __launch_bounds__(256) mtrt_dq_##KN##_##XN##_##QN(                                    \
      const QT::storage* q, XT::storage* y, const float* scale, int64_t n, int64_t d1, int64_t nb, int64_t fpitch, \
      int64_t qpitch) { qdq_rows_ragged<XT, QT, KIND, 1>(nullptr, const_cast<QT::storage*>(q), y, scale, n, d1, nb, fpitch, qpitch, 0); } \
  extern "C" __global__ void __launch_bounds__(256) mtrt_qdq_##KN##_##XN##_##QN(                                   \
      const XT::storage* x, QT::storage* q, XT::storage* y, const float* scale, int64_t n, int64_t d1, int64_t nb, \
      int64_t fpitch, int64_t qpitch, int32_t flags) { qdq_rows_ragged<XT, QT, KIND, 2>(x, q, y, scale, n, d1, nb, fpitch, qpitch, flags); }
#define MTRT_QDQ_RAGGED_FOR_FLOAT(XN, XT)                                                                          \
  MTRT_QDQ_RAGGED_KERNELS(XN, XT, i8, I8, rowu, kRow) MTRT_QDQ_RAGGED_KERNELS(XN, XT, i8, I8, colu, kCol)          \
  MTRT_QDQ_RAGGED_KERNELS(XN, XT, f8, F8, rowu, kRow) MTRT_QDQ_RAGGED_KERNELS(XN, XT, f8, F8, colu, kCol)          \
  MTRT_QDQ_RAGGED_KERNELS(XN, XT, i4, I4, rowu, kRow) MTRT_QDQ_RAGGED_KERNELS(XN, XT, i4, I4, colu, kCol)
MTRT_QDQ_RAGGED_FOR_FLOAT(f32, F32)
MTRT_QDQ_RAGGED_FOR_FLOAT(f16, F16)
MTRT_QDQ_RAGGED_FOR_FLOAT(bf16, BF16)

// ---- strided views ------------------------------------------------------------------
// The same element-wise programs on rank-2 VIEWS: each tensor operand arrives as the reference expands a fully
// dynamic memref<?x?xT, strided<[?, ?], offset: ?>> argument (mlir-tensorrt/kernel/lib/Kernel/Transforms/
// ExpandMemRefArgs.cpp:65-120; operand order pinned by mlir-tensorrt/compiler/test/Passes/1_Core/KernelToCUDA/
// kernel-to-cuda.mlir:3-48): aligned base pointer, offset, size 0, size 1, stride 0, stride 1, all in elements as
// 64-bit integers; element (r, c) lives at base[offset + r * stride0 + c * stride1].  The scale is a contiguous
// constant addressed by the LOGICAL (r, c) of the view: uniform scale[0], row scale[r % nb], col
// scale[(r / nb) * size1 + c].  One element per lane; codes one per byte (i8, f8E4M3FN, int4 in the low nibble).
namespace qdq_cluster {

template <typename X, typename Q, int MODE>   // MODE 0: quantize x -> q ; 1: dequantize q -> x
__device__ __forceinline__ void qdq_view(typename X::storage* __restrict__ xb, int64_t xo, int64_t xs0, int64_t xs1,
                                         typename Q::storage* __restrict__ qb, int64_t qo, int64_t qs0, int64_t qs1,
                                         const float* __restrict__ scale, int64_t d0, int64_t d1, int64_t nb, int kind, int flags) {
  const int64_t n = d0 * d1;
  const int64_t stride = int64_t(gridDim.x) * blockDim.x;
  for (int64_t e = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; e < n; e += stride) {
    const int64_t r = e / d1, c = e - r * d1;
    const float s = kind == kUniform ? scale[0] : (kind == kRow ? scale[r % nb] : scale[(r / nb) * d1 + c]);
    typename X::storage* xp = xb + xo + r * xs0 + c * xs1;
    typename Q::storage* qp = qb + qo + r * qs0 + c * qs1;
    if (MODE == 0) {
      const float v = quant_value<Q>(Tile<X>::load1(xp), s, flags);
      *qp = typename Q::storage(Codes<Q>::enc(v, flags));
    } else {
      Tile<X>::store1(xp, Codes<Q>::dec(uint32_t(uint8_t(*qp))) * s);
    }
  }
}

// The same program in 64 x 64 tiles through LDS, for views whose operands run fastest along different dimensions (a
// transposed source into a row-major destination and the like): one element per lane moves a few bytes per cache
// line on the side it walks against the grain (f16 [8192, 8192] transposed to i8: 0.9 TB/s).  Here each side is
// walked along its own fastest dimension: the source side fills the tile (floats, or decoded codes), the
// destination side empties it, applying the scale of the element's logical (r, c).  The pitch of 65 floats keeps
// both walks free of bank conflicts.  Grid: any (tiles are dealt round-robin), block = 256.
template <typename X, typename Q, int MODE>
__device__ __forceinline__ void qdq_view_tiles(typename X::storage* __restrict__ xb, int64_t xo, int64_t xs0, int64_t xs1,
                                               typename Q::storage* __restrict__ qb, int64_t qo, int64_t qs0, int64_t qs1,
                                               const float* __restrict__ scale, int64_t d0, int64_t d1, int64_t nb, int kind,
                                               int flags) {
  __shared__ float tile[64][65];
  auto magnitude = [](int64_t v) { return v < 0 ? -v : v; };
  const bool x_d0_fast = magnitude(xs0) < magnitude(xs1), q_d0_fast = magnitude(qs0) < magnitude(qs1);
  const bool src_d0_fast = MODE == 0 ? x_d0_fast : q_d0_fast, dst_d0_fast = MODE == 0 ? q_d0_fast : x_d0_fast;
  const int64_t tiles_c = (d1 + 63) / 64, tiles = ((d0 + 63) / 64) * tiles_c;
  const int a = threadIdx.x & 63, b0 = threadIdx.x >> 6;
  for (int64_t t = blockIdx.x; t < tiles; t += gridDim.x) {
    const int64_t r0 = (t / tiles_c) * 64, c0 = (t % tiles_c) * 64;
#pragma unroll 4
    for (int i = 0; i < 16; ++i) {
      const int b = b0 + 4 * i;
      const int lr = src_d0_fast ? a : b, lc = src_d0_fast ? b : a;
      const int64_t r = r0 + lr, c = c0 + lc;
      if (r < d0 && c < d1)
        tile[lr][lc] = MODE == 0 ? Tile<X>::load1(xb + xo + r * xs0 + c * xs1)
                                 : Codes<Q>::dec(uint32_t(uint8_t(qb[qo + r * qs0 + c * qs1])));
    }
    __syncthreads();
#pragma unroll 4
    for (int i = 0; i < 16; ++i) {
      const int b = b0 + 4 * i;
      const int lr = dst_d0_fast ? a : b, lc = dst_d0_fast ? b : a;
      const int64_t r = r0 + lr, c = c0 + lc;
      if (r < d0 && c < d1) {
        const float s = kind == kUniform ? scale[0] : (kind == kRow ? scale[r % nb] : scale[(r / nb) * d1 + c]);
        if (MODE == 0) {
          const float v = quant_value<Q>(tile[lr][lc], s, flags);
          qb[qo + r * qs0 + c * qs1] = typename Q::storage(Codes<Q>::enc(v, flags));
        } else {
          Tile<X>::store1(xb + xo + r * xs0 + c * xs1, tile[lr][lc] * s);
        }
      }
    }
    __syncthreads();
  }
}

}  // namespace qdq_cluster

//   q_view  (x: base, offset, size0, size1, stride0, stride1 ; q: the same six ; scale, nb, kind, flags)
//   dq_view (q: six ; y: six ; scale, nb, kind)
// The two operands of a call have equal sizes; the kernel reads them from the first one.  The _viewt_ forms take the
// same arguments and walk 64 x 64 tiles (see qdq_view_tiles).
#define MTRT_QDQ_VIEW_KERNELS(XN, XT, QN, QT)                                                                        \
  extern "C" __global__ void __launch_bounds__(256) mtrt_q_view_##XN##_##QN(                                         \
      const XT::storage* x, int64_t xo, int64_t d0, int64_t d1, int64_t xs0, int64_t xs1, QT::storage* q, int64_t qo, \
      int64_t, int64_t, int64_t qs0, int64_t qs1, const float* scale, int64_t nb, int32_t kind, int32_t flags) {     \
    qdq_view<XT, QT, 0>(const_cast<XT::storage*>(x), xo, xs0, xs1, q, qo, qs0, qs1, scale, d0, d1, nb, kind, flags); } \
  extern "C" __global__ void __launch_bounds__(256) mtrt_dq_view_##XN##_##QN(                                        \
      const QT::storage* q, int64_t qo, int64_t d0, int64_t d1, int64_t qs0, int64_t qs1, XT::storage* y, int64_t yo, \
      int64_t, int64_t, int64_t ys0, int64_t ys1, const float* scale, int64_t nb, int32_t kind) {                    \
    qdq_view<XT, QT, 1>(y, yo, ys0, ys1, const_cast<QT::storage*>(q), qo, qs0, qs1, scale, d0, d1, nb, kind, 0); }   \
  extern "C" __global__ void __launch_bounds__(256) mtrt_q_viewt_##XN##_##QN(                                        \
      const XT::storage* x, int64_t xo, int64_t d0, int64_t d1, int64_t xs0, int64_t xs1, QT::storage* q, int64_t qo, \
      int64_t, int64_t, int64_t qs0, int64_t qs1, const float* scale, int64_t nb, int32_t kind, int32_t flags) {     \
    qdq_view_tiles<XT, QT, 0>(const_cast<XT::storage*>(x), xo, xs0, xs1, q, qo, qs0, qs1, scale, d0, d1, nb, kind, flags); } \
  extern "C" __global__ void __launch_bounds__(256) mtrt_dq_viewt_##XN##_##QN(                                       \
      const QT::storage* q, int64_t qo, int64_t d0, int64_t d1, int64_t qs0, int64_t qs1, XT::storage* y, int64_t yo, \
      int64_t, int64_t, int64_t ys0, int64_t ys1, const float* scale, int64_t nb, int32_t kind) {                    \
    qdq_view_tiles<XT, QT, 1>(y, yo, ys0, ys1, const_cast<QT::storage*>(q), qo, qs0, qs1, scale, d0, d1, nb, kind, 0); }
#define MTRT_QDQ_VIEW_FOR_X(XN, XT)  \
  MTRT_QDQ_VIEW_KERNELS(XN, XT, i8, I8) MTRT_QDQ_VIEW_KERNELS(XN, XT, f8, F8) MTRT_QDQ_VIEW_KERNELS(XN, XT, i4, I4)
MTRT_QDQ_VIEW_FOR_X(f32, F32)
MTRT_QDQ_VIEW_FOR_X(f16, F16)
MTRT_QDQ_VIEW_FOR_X(bf16, BF16)
