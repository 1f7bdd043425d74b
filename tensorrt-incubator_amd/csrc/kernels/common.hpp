// Device-side building blocks shared by the gfx950 kernels of this module:
// 128-bit global accesses, wave64 reductions, and the narrow-type conversions
// whose results must equal the CPU restatement of the reference's host number
// classes (mlir-tensorrt/executor/lib/Runtime/Backend/Common/DataTypes.cpp:43-519).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mtrt_dev {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

// Element-type tags.  `storage` is what lives in HBM; kBits is bits per element.
struct F32 { using storage = float;    static constexpr int kBits = 32; };
struct F16 { using storage = uint16_t; static constexpr int kBits = 16; };
struct BF16 { using storage = uint16_t; static constexpr int kBits = 16; };
struct I8 { using storage = int8_t;    static constexpr int kBits = 8; };
struct F8 { using storage = uint8_t;   static constexpr int kBits = 8; };
struct I4 { using storage = uint8_t;   static constexpr int kBits = 8; };  // one per byte, low nibble
struct I4P { using storage = uint8_t;  static constexpr int kBits = 4; };  // two per byte, even index low
struct F4P { using storage = uint8_t;  static constexpr int kBits = 4; };  // f4E2M1FN, two per byte, even index low

// flag bits passed by value to the quantize kernels
constexpr int kFlagRoundToInt = 1;   // round_nearest_even before the clamp (f8 target only; ints always round)
constexpr int kFlagF8RefHost = 2;    // reproduce the reference host class instead of IEEE RNE+saturate
constexpr int kFlagF8ViaF16 = 4;     // f32 -> f16 -> f8, both RNE: the conversion chain of the reference's GPU path

__device__ __forceinline__ float bits_to_f32(uint32_t u) { return __uint_as_float(u); }
__device__ __forceinline__ uint32_t f32_to_bits(float f) { return __float_as_uint(f); }

// ---- widening (exact) -------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return bits_to_f32(b << 16); }
__device__ __forceinline__ float f16_bits_to_f32(uint32_t b) {
  union { uint16_t u; _Float16 h; } c;
  c.u = uint16_t(b);
  return float(c.h);
}
// ---- narrowing, IEEE round-to-nearest-even ----------------------------------
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  union { __bf16 h; uint16_t u; } c;
  c.h = (__bf16)f;                       // v_cvt_pk_bf16_f32: RNE, NaN quieted
  return c.u;
}
__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  // The empty asm hides how `f` was produced.  Without it the compiler merges a
  // preceding f32 multiply/add into v_fma_mixlo_f16, which rounds the exact result
  // to f16 ONCE; the host program rounds to f32 first and then to f16, and the two
  // differ whenever the f32 rounding lands on an f16 tie.
  __asm__("" : "+v"(f));
  union { _Float16 h; uint16_t u; } c;
  c.h = (_Float16)f;                     // v_cvt_f16_f32: RNE, overflow -> inf, subnormals kept
  return c.u;
}
// Two at once into one word (lo in bits 0..15): v_cvt_pk_f16_f32, the same rounding; half the instructions of
// two single conversions and no merge of the halves.
__device__ __forceinline__ uint32_t f32x2_to_f16x2_bits(float lo, float hi) {
  __asm__("" : "+v"(lo), "+v"(hi));      // as above: no merging of the producers into a single rounding
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
  union { f16x2_t h; uint32_t u; } c;
  c.h = __builtin_convertvector((f32x2_t){lo, hi}, f16x2_t);
  return c.u;
}
__device__ __forceinline__ uint32_t f32x2_to_bf16x2_bits(float lo, float hi) {
  return f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
}

// f8E4M3FN (OCP) pair conversion in hardware: RNE.  Inputs are pre-clamped to
// [-448, 448] by every caller, so the saturation rule of the instruction is
// never exercised.
__device__ __forceinline__ uint32_t f32x2_to_f8_ieee(float a, float b) {
  return uint32_t(__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false)) & 0xFFFFu;
}

// f8E4M3FN exactly as the reference HOST class computes it
// (DataTypes.cpp:43-122), valid for |v| <= 448 and non-NaN v.  Differences
// from IEEE, all reproduced here:
//   - results that IEEE-round to 256..448 (biased exponent 15) become +-448;
//   - in the subnormal range (|v| < 2^-6) the 24-bit significand is shifted
//     right first, dropping the shifted-out bits, then rounded on 20 guard bits;
//   - a subnormal that rounds up to 8/8 loses the carry and becomes +-0.
__device__ __forceinline__ uint32_t f32_to_f8_refhost(float v) {
  const uint32_t u = f32_to_bits(v);
  const uint32_t sign = (u >> 24) & 0x80u;
  const uint32_t e32 = (u >> 23) & 0xFFu;
  const uint32_t m32 = u & 0x7FFFFFu;
  const int e = int(e32) - 120;                      // biased f8 exponent
  if (e32 == 0) return sign;                         // zero / f32 subnormal
  if (e >= 15) return sign | 0x7Eu;
  if (e >= 1) {
    uint32_t mag = (uint32_t(e) << 3) | (m32 >> 20);
    const uint32_t rem = m32 & 0xFFFFFu;
    mag += (rem > 0x80000u || (rem == 0x80000u && (mag & 1u))) ? 1u : 0u;
    return (mag >= 0x78u) ? (sign | 0x7Eu) : (sign | mag);
  }
  if (e < -3) return sign;
  const uint32_t shifted = (m32 | 0x800000u) >> uint32_t(1 - e);
  uint32_t keep = shifted >> 20;
  const uint32_t rem = shifted & 0xFFFFFu;
  keep += (rem > 0x80000u || (rem == 0x80000u && (keep & 1u))) ? 1u : 0u;
  return sign | (keep & 7u);
}

// f8E4M3FN -> f32, exact (DataTypes.cpp:124-174).  gfx950 converts OCP fp8 in
// hardware; `sel` picks the byte of the packed word.
template <int SEL>
__device__ __forceinline__ float f8_to_f32(uint32_t packed) {
  return __builtin_amdgcn_cvt_f32_fp8(int(packed), SEL);
}

// ---- wave / block reductions ------------------------------------------------
template <typename T, typename Op>
__device__ __forceinline__ T wave_reduce(T v, Op op) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1)
    v = op(v, __shfl_xor(v, off, kWave));
  return v;
}
struct MaxU32 { __device__ __forceinline__ uint32_t operator()(uint32_t a, uint32_t b) const { return a > b ? a : b; } };
struct MaxF32 { __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); } };
struct SumF32 { __device__ __forceinline__ float operator()(float a, float b) const { return a + b; } };

// ---- single-element access ------------------------------------------------------
constexpr int kTile = 16;            // elements a lane carries per trip in the elementwise kernels

template <typename T> struct Tile;   // load1 / store1: one element <-> f32

template <> struct Tile<F32> {
  static __device__ __forceinline__ float load1(const float* p) { return *p; }
  static __device__ __forceinline__ void store1(float* p, float v) { *p = v; }
};

template <> struct Tile<BF16> {
  static __device__ __forceinline__ float load1(const uint16_t* p) { return bf16_bits_to_f32(*p); }
  static __device__ __forceinline__ void store1(uint16_t* p, float v) { *p = uint16_t(f32_to_bf16_bits(v)); }
};

template <> struct Tile<F16> {
  static __device__ __forceinline__ float load1(const uint16_t* p) { return f16_bits_to_f32(*p); }
  static __device__ __forceinline__ void store1(uint16_t* p, float v) { *p = uint16_t(f32_to_f16_bits(v)); }
};

}  // namespace mtrt_dev
