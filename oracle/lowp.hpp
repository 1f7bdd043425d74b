// TEST INFRASTRUCTURE — CPU oracle, not a product path.
//
// Software conversions between f32 and the narrow storage types the
// quantization path uses (f8E4M3FN, f16, bf16, int4).  This is a restatement
// of the *behaviour* of the reference executor's host number classes
//   mlir-tensorrt/executor/lib/Runtime/Backend/Common/DataTypes.cpp:43-122   (f32 -> f8E4M3FN)
//   mlir-tensorrt/executor/lib/Runtime/Backend/Common/DataTypes.cpp:124-174  (f8E4M3FN -> f32)
//   mlir-tensorrt/executor/lib/Runtime/Backend/Common/DataTypes.cpp:226-306  (f32 -> f16)
//   mlir-tensorrt/executor/lib/Runtime/Backend/Common/DataTypes.cpp:308-359  (f16 -> f32)
//   mlir-tensorrt/executor/lib/Runtime/Backend/Common/DataTypes.cpp:411-442  (bf16 both ways)
//   mlir-tensorrt/executor/lib/Runtime/Backend/Common/DataTypes.cpp:494-519  (int4 saturate / sign-extend)
// written as ONE parameterised narrowing routine instead of one routine per
// type, with two selectable behaviours:
//
//   kIeee    : IEEE-754 round-to-nearest-even narrowing; f8E4M3FN saturates to
//              +-448 (no infinity), NaN -> canonical NaN.  This equals the
//              reference GPU path's `cvt.rn.satfinite` and the gfx950 hardware
//              conversion, and is what "round-half-to-even with saturation"
//              means.
//   kRefHost : bit-for-bit what the reference's host classes return, including
//              their three deviations from IEEE:
//                (1) f8: a biased exponent of 15 is treated as overflow, so every
//                    |x| that would round to 256..448 becomes +-448;
//                (2) f8/f16: a subnormal that rounds up to the smallest normal
//                    loses its carry and becomes +-0;
//                (3) f8/f16: in the subnormal range the bits shifted out before
//                    the guard field is taken are dropped (no sticky), so a
//                    value just above a tie is rounded as if it were the tie.
//              and (4) bf16: a NaN whose rounding increment overflows the
//                    exponent field (0x7FFFxxxx with round-up) wraps to -0/+0.
//
// Pinning: every function here is checked (a) exhaustively over all 2^32 f32
// inputs against the compiled reference file (oracle/_ref, `make -C oracle pin`),
// (b) against committed golden tables minted from that build, (c) kIeee against
// numpy float16 / torch bfloat16 / torch float8_e4m3fn casts, and (d) against the
// known answers in the reference's own tests (see tests/test_oracle_lowp.py).
#pragma once
#include <cstdint>
#include <cstring>

namespace orc {

enum ConvMode : int { kIeee = 0, kRefHost = 1 };

inline uint32_t f32_bits(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  return u;
}
inline float bits_f32(uint32_t u) {
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

// Narrow an f32 to a sign/EBITS/MBITS format with bias 2^(EBITS-1)-1.
//   HAS_INF : top exponent is reserved for inf/NaN (f16).  Otherwise the format
//             is "FN": only the all-ones pattern is NaN and there is no inf (f8).
template <int EBITS, int MBITS, bool HAS_INF>
inline uint32_t narrow_f32(float value, ConvMode mode) {
  constexpr int kBias = (1 << (EBITS - 1)) - 1;
  constexpr int kDrop = 23 - MBITS;                       // f32 mantissa bits dropped
  constexpr uint32_t kExpAll = (1u << EBITS) - 1;
  constexpr uint32_t kMagMask = (1u << (EBITS + MBITS)) - 1;
  constexpr uint32_t kInf = kExpAll << MBITS;             // only if HAS_INF
  constexpr uint32_t kNaN = HAS_INF ? (kInf | (1u << (MBITS - 1))) : kMagMask;
  constexpr uint32_t kMaxFinite = HAS_INF ? (kInf - 1) : (kMagMask - 1);

  const uint32_t u = f32_bits(value);
  const uint32_t sign = (u >> 31) << (EBITS + MBITS);
  const uint32_t e32 = (u >> 23) & 0xFF;
  const uint32_t m32 = u & 0x7FFFFF;

  if (e32 == 0xFF) {
    if (m32 != 0)
      return HAS_INF ? (sign | kNaN) : kNaN;              // ref f8: NaN is 0x7F, sign dropped
    if (HAS_INF)
      return sign | kInf;
    return sign | kMaxFinite;                             // f8: +-inf saturates
  }
  if (e32 == 0 && m32 == 0)
    return sign;
  // f32 subnormals are far below every narrow format's range: e below is very
  // negative and the subnormal branch returns a signed zero.
  const int e = int(e32) - 127 + kBias;                   // biased exponent in the narrow format

  if (e >= 1) {
    if (mode == kRefHost && !HAS_INF && e >= int(kExpAll))
      return sign | kMaxFinite;                           // deviation (1), pre-rounding
    if (e >= int(kExpAll) + (HAS_INF ? 0 : 1))
      return sign | (HAS_INF ? kInf : kMaxFinite);
    uint32_t keep = m32 >> kDrop;
    const uint32_t rem = m32 & ((1u << kDrop) - 1);
    const uint32_t half = 1u << (kDrop - 1);
    uint32_t mag = (uint32_t(e) << MBITS) | keep;
    if (rem > half || (rem == half && (keep & 1)))
      mag += 1;                                           // carry may bump the exponent
    if (mode == kRefHost && !HAS_INF && (mag >> MBITS) >= kExpAll)
      return sign | kMaxFinite;                           // deviation (1), post-rounding
    if (mag > kMaxFinite)
      return sign | (HAS_INF ? kInf : kMaxFinite);
    return sign | mag;
  }

  // Subnormal (or underflow) in the narrow format.
  const int shift = 1 - e;                                // >= 1
  if (shift > MBITS + 1 && mode == kRefHost)
    return sign;                                          // ref: "too small even for denormal"
  if (shift > 24)
    return sign;                                          // below half of the least subnormal
  const uint32_t full = m32 | 0x800000;
  if (mode == kRefHost) {
    const uint32_t shifted = full >> shift;               // deviation (3): bits fall off here
    uint32_t keep = shifted >> kDrop;
    const uint32_t rem = shifted & ((1u << kDrop) - 1);
    const uint32_t half = 1u << (kDrop - 1);
    if (rem > half || (rem == half && (keep & 1)))
      keep += 1;
    return sign | (keep & ((1u << MBITS) - 1));           // deviation (2): carry masked off
  }
  const int total = kDrop + shift;                        // <= kDrop + 24 < 64
  const uint64_t wide = full;
  uint32_t keep = total >= 32 ? 0u : uint32_t(wide >> total);
  const uint64_t rem = wide & ((uint64_t(1) << total) - 1);
  const uint64_t half = uint64_t(1) << (total - 1);
  if (rem > half || (rem == half && (keep & 1)))
    keep += 1;                                            // may become the least normal: correct
  return sign | keep;
}

// Widen a sign/EBITS/MBITS value to f32 (exact).
template <int EBITS, int MBITS, bool HAS_INF>
inline float widen_to_f32(uint32_t bits) {
  constexpr int kBias = (1 << (EBITS - 1)) - 1;
  constexpr uint32_t kExpAll = (1u << EBITS) - 1;
  constexpr uint32_t kMagMask = (1u << (EBITS + MBITS)) - 1;
  const uint32_t sign = ((bits >> (EBITS + MBITS)) & 1u) << 31;
  const uint32_t e = (bits >> MBITS) & kExpAll;
  uint32_t m = bits & ((1u << MBITS) - 1);
  if (HAS_INF && e == kExpAll)
    return bits_f32(sign | (m ? 0x7FC00000u : 0x7F800000u));
  if (!HAS_INF && (bits & kMagMask) == kMagMask)
    return bits_f32(0x7FC00000u);                         // ref: positive quiet NaN
  if (e == 0) {
    if (m == 0)
      return bits_f32(sign);
    int lead = MBITS - 1;                                 // index of the leading one
    while (!((m >> lead) & 1))
      --lead;
    const int exp32 = 127 - kBias + 1 - (MBITS - lead);
    m = (m << (MBITS - lead)) & ((1u << MBITS) - 1);
    return bits_f32(sign | (uint32_t(exp32) << 23) | (m << (23 - MBITS)));
  }
  return bits_f32(sign | ((e - kBias + 127) << 23) | (m << (23 - MBITS)));
}

inline uint8_t f32_to_f8e4m3fn(float x, ConvMode mode) {
  return uint8_t(narrow_f32<4, 3, false>(x, mode));
}
inline float f8e4m3fn_to_f32(uint8_t b) { return widen_to_f32<4, 3, false>(b); }

inline uint16_t f32_to_f16(float x, ConvMode mode) {
  return uint16_t(narrow_f32<5, 10, true>(x, mode));
}
inline float f16_to_f32(uint16_t b) { return widen_to_f32<5, 10, true>(b); }

// bf16 keeps the f32 exponent, so narrowing is a rounding of the bit pattern.
inline uint16_t f32_to_bf16(float x, ConvMode mode) {
  const uint32_t u = f32_bits(x);
  const bool is_nan = ((u & 0x7F800000u) == 0x7F800000u) && (u & 0x7FFFFFu);
  if (mode == kIeee && is_nan)
    return uint16_t((u >> 16) | 0x0040u);                 // quiet, payload/sign kept
  uint32_t hi = u >> 16;
  const uint32_t low = u & 0xFFFFu;
  if (low > 0x8000u || (low == 0x8000u && (hi & 1)))
    hi += 1;                                              // inf stays inf; max finite -> inf
  if (mode == kRefHost && (hi & 0x7F80u) == 0x7F80u && (u & 0x7FFFFFu))
    hi |= 0x0040u;                                        // deviation (4) lives in the `hi += 1` above
  return uint16_t(hi);
}
inline float bf16_to_f32(uint16_t b) { return bits_f32(uint32_t(b) << 16); }

// int4: construction from an int saturates to [-8, 7]; reading sign-extends the
// low nibble (DataTypes.cpp:494-519).
inline int8_t int4_saturate(int v) { return int8_t(v > 7 ? 7 : (v < -8 ? -8 : v)); }
inline int8_t int4_sign_extend(uint8_t nibble) {
  return int8_t((nibble & 0x8) ? (nibble | 0xF0) : (nibble & 0xF));
}

// f4E2M1FN (values 0, 0.5, 1, 1.5, 2, 3, 4, 6 with a sign bit; no inf, no NaN) from f16, restating
// the executor's expansion of `truncf f16 -> f4E2M1FN`
// (mlir-tensorrt/executor/lib/Passes/ExpandOps.cpp:471-694): classification by f16 exponent and
// mantissa thresholds, which is round-to-nearest-even with saturation to +-6; inf -> +-6, NaN -> 0.
// kRefHost keeps the expansion's treatment of zero: an f16 that is exactly +-0 gives code 0 (the
// sign is dropped, :687), while a negative f16 subnormal gives code 8 (-0).  kIeee keeps the sign
// of zero in both cases (what a hardware conversion does).
inline uint8_t f16_to_f4e2m1fn(uint16_t h, ConvMode mode) {
  const uint32_t sign = (h >> 15) & 1u, exp = (h >> 10) & 0x1Fu, mant = h & 0x3FFu;
  if (exp == 31)
    return mant ? 0 : uint8_t(sign ? 15 : 7);
  if (mode == kRefHost && exp == 0 && mant == 0)
    return 0;
  uint32_t code;
  if (exp < 13) code = 0;
  else if (exp == 13) code = mant == 0 ? 0 : 1;            // 0.25 ties to 0
  else if (exp == 14) code = mant < 512 ? 1 : 2;           // 0.75 ties to 1.0
  else if (exp == 15) code = mant <= 256 ? 2 : (mant < 768 ? 3 : 4);
  else if (exp == 16) code = mant <= 256 ? 4 : (mant < 768 ? 5 : 6);
  else if (exp == 17) code = mant <= 256 ? 6 : 7;          // 5.0 ties to 4.0
  else code = 7;
  return uint8_t(code | (sign << 3));
}
// exact widening (ExpandOps.cpp:365-461 goes f4 -> f16; every value is representable)
inline float f4e2m1fn_to_f32(uint8_t code) {
  static const float kMag[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
  const float v = kMag[code & 7];
  return (code & 8) ? -v : v;
}

} // namespace orc
