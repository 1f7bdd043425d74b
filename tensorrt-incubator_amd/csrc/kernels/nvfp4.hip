// NVFP4 block quantize / dequantize for gfx950: the two-level scaling of tensorrt.dynamic_quantize
// (mlir-tensorrt/tensorrt/include/mlir-tensorrt-dialect/TensorRT/IR/TensorRTOps.td:3279-3358) in the
// program form of mlir-tensorrt/integrations/PJRT/test/JAX/test_q_dq_nvfp4.py:21-45, blocks of 16
// along the last axis (or, in the *_cols kernels at the end, the second-to-last), every op in f32 and in this order:
//     S_dec_x = max|x_block| / 6        S_enc = 2688 / tensor_amax
//     s8      = f8e4m3fn(S_dec_x * S_enc)                  (block scale, stored)
//     S_enc_x = S_enc / f32(s8)         q = f4e2m1fn(f16(x * S_enc_x))
//     y       = narrow(f32(q) * (f32(s8) * (tensor_amax / 2688)))
// Conversions to f4 go through f16, the only f4 truncation the reference defines (RNE, saturation
// to +-6, inf -> +-6, NaN -> 0: mlir-tensorrt/executor/lib/Passes/ExpandOps.cpp:471-694).  An all-zero
// block has s8 = 0, S_enc_x = inf and x * S_enc_x = NaN, which that conversion maps to code 0; the
// same chain is evaluated here, no block is special-cased.  Only the last step differs by value: the
// hardware conversion gives a NaN another code than the reference's table, so NaN products take the table.
//
// Data movement: as in the quantize/dequantize clusters a lane owns one 128-bit vector of the float
// operand per trip (4 f32 or 8 f16/bf16), so a block of 16 is held by 4 (or 2) neighbouring lanes
// and its amax is two (one) cross-lane exchanges; every lane of the block then evaluates the
// block's scalar chain itself.  A wave handles 8 consecutive trips (8 KiB of the float operand);
// its codes (1 or 2 KiB) and block scales (128 or 256 B) are parked in the wave's own LDS region
// and written out as whole cache lines, 16 bytes per lane.
#include "common.hpp"

namespace nvfp4_cluster {

using namespace mtrt_dev;
using qdq_cluster::FloatGroup;

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef float f2 __attribute__((ext_vector_type(2)));

constexpr int kThreads = 256;
constexpr int kTrips = 8;

// the reference's table on one f16 bit pattern (exact, slow): used for blocks that contain NaN
__device__ __forceinline__ uint32_t f16_bits_to_f4_exact(uint32_t h) {
  const uint32_t a = h & 0x7FFFu, sign = (h >> 12) & 8u;
  if (a > 0x7C00u) return 0;
  const uint32_t code = (a > 0x3400u) + (a >= 0x3A00u) + (a > 0x3D00u) + (a >= 0x3F00u) + (a > 0x4100u) + (a >= 0x4300u) +
                        (a > 0x4500u);
  return code | sign;
}
// G products -> G f16 values (RNE), two per word, product k in half k % 2 of word k / 2
template <int G>
__device__ __forceinline__ void products_to_f16(float (&w)[G], uint32_t (&h)[G / 2]) {
#pragma unroll
  for (int k = 0; k < G; k += 2) {
    // The empty asm keeps the products' own f32 rounding in front of the f16 rounding (see f32_to_f16_bits in
    // common.hpp: without it the multiply and the conversion merge into one instruction that rounds once).
    __asm__("" : "+v"(w[k]), "+v"(w[k + 1]));
    union { h2 v; uint32_t u; } c;
    c.v = (h2){(_Float16)w[k], (_Float16)w[k + 1]};
    h[k / 2] = c.u;
  }
}
// is any of the G values a NaN?  (one unordered compare per pair)
template <int G>
__device__ __forceinline__ bool any_nan(const float (&w)[G]) {
  bool r = false;
#pragma unroll
  for (int k = 0; k < G; k += 2) r = r || __builtin_isunordered(w[k], w[k + 1]);
  return r;
}
// G f16 values -> G f4E2M1FN codes, value k in nibble k: the hardware conversion writes one byte of its
// destination and keeps the others.  Right for ordinary values; NaN (code 0 by the reference's rule) is
// patched in by the caller per block.
template <int G>
__device__ __forceinline__ uint32_t f16_to_f4(const uint32_t (&h)[G / 2]) {
  union { uint32_t u; h2 v; } c;
  c.u = h[0];
  uint32_t codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(0u, c.v, 1.0f, 0);
  c.u = h[1];
  codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(codes, c.v, 1.0f, 1);
  if (G == 8) {
    c.u = h[2 % (G / 2)];
    codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(codes, c.v, 1.0f, 2);
    c.u = h[3 % (G / 2)];
    codes = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(codes, c.v, 1.0f, 3);
  }
  return codes;
}
// the reference's table on value k of the packed f16 words
template <int G>
__device__ __forceinline__ uint32_t f16_to_f4_exact(const uint32_t (&h)[G / 2], int k) {
  return f16_bits_to_f4_exact((h[k / 2] >> (16 * (k & 1))) & 0xFFFFu);
}
// x / 6 for x >= 0 (a block maximum), correctly rounded, in 5 instructions instead of the 11 of the IEEE divide
// expansion: q0 = RN(x r), q = RN(q0 + RN(x - 6 q0) r) with r = RN(1/6) (the remainder of a faithful quotient is
// exact in an FMA; Markstein's correction).  Compared with the IEEE quotient on EVERY non-negative f32 on the
// CPU: equal for +0 and for all of [2^-125, FLT_MAX]; below (the remainder is no longer exact) and for
// inf / NaN the lanes take the real divide, in a wave-uniform branch that ordinary data never enters.
__device__ __forceinline__ float divide_by_six(float x) {
  const float r = 1.0f / 6.0f;
  const float q0 = x * r;
  float q = __builtin_fmaf(__builtin_fmaf(-q0, 6.0f, x), r, q0);
  // x / 2 is exact, and a positive normal number or +0 exactly where the short form holds: any other class
  // (0x2BF = all ten classes but those two) takes the divide
  const bool other = __builtin_amdgcn_classf(x * 0.5f, 0x2BF);
  if (__builtin_amdgcn_ballot_w64(other) != 0) q = other ? x / 6.0f : q;
  return q;
}
// S_enc / f32(s8) for every scale byte, one IEEE divide per lane of the workgroup (256 lanes): a block's second
// divide becomes a look-up.  Every lane of the workgroup must get here (there is a barrier inside).
__device__ __forceinline__ void fill_inverse_scales(float* table, float s_enc) {
  for (uint32_t b = threadIdx.x; b < 256u; b += blockDim.x) table[b] = s_enc / f8_to_f32<0>(b);
  __syncthreads();
}

// (x, q_packed, scales, tensor_amax, nvec) ; nvec 128-bit vectors of x, a multiple of the vectors per block
template <typename X>
__device__ __forceinline__ void quantize_body(const typename X::storage* __restrict__ x, uint8_t* __restrict__ q,
                                              uint8_t* __restrict__ scales, const float* __restrict__ tensor_amax,
                                              int64_t nvec) {
  constexpr int G = FloatGroup<X>::G;                  // elements per vector: 4 or 8
  constexpr int LPB = 16 / G;                          // lanes per block: 4 or 2
  constexpr int kCodeBytes = G / 2;                    // code bytes per lane and trip
  constexpr int kSpanCodes = kTrips * 64 * kCodeBytes; // 1 or 2 KiB per wave
  constexpr int kSpanScales = kTrips * 64 / LPB;       // 128 or 256 B per wave
  __shared__ __attribute__((aligned(16))) uint8_t lds[(kThreads / 64) * (kSpanCodes + kSpanScales)];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint8_t* my_codes = lds + wave * (kSpanCodes + kSpanScales);
  uint8_t* my_scales = my_codes + kSpanCodes;
  __shared__ float inverse_scale[256];
  const int64_t span = (int64_t(blockIdx.x) * (kThreads / 64) + wave) * (kTrips * 64);   // first vector of this wave
  const float s_enc = 2688.0f / *tensor_amax;
  fill_inverse_scales(inverse_scale, s_enc);
  if (span >= nvec) return;                            // whole wave

  u32x4 t[kTrips];
#pragma unroll
  for (int j = 0; j < kTrips; ++j) {
    int64_t v = span + j * 64 + lane;
    v = v < nvec ? v : nvec - 1;                       // past the end: a valid vector, its results are not stored
    t[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(x) + v);
  }
#pragma unroll
  for (int j = 0; j < kTrips; ++j) {
    float v[G];
    FloatGroup<X>::unpack(t[j], v);
    float amax = 0.0f;
#pragma unroll
    for (int k = 0; k < G; ++k) amax = fmaxf(amax, fabsf(v[k]));
#pragma unroll
    for (int off = 1; off < LPB; off <<= 1) amax = fmaxf(amax, __shfl_xor(amax, off, kWave));
    const float s_dec_x = divide_by_six(amax);
    uint32_t s8 = f32x2_to_f8_ieee(s_dec_x * s_enc, 0.0f) & 0xFFu;
    s8 = (s8 & 0x7Fu) == 0x7Fu ? 0x7Fu : s8;             // NaN (0 * inf when the tensor amax is 0): 0x7F whatever its sign, as the host class
    const float s_enc_x = inverse_scale[s8];             // = s_enc / f32(s8), the same IEEE quotient
    float w[G];
#pragma unroll
    for (int k = 0; k < G; ++k) w[k] = v[k] * s_enc_x;
    uint32_t h[G / 2];
    products_to_f16<G>(w, h);
    uint32_t codes = f16_to_f4<G>(h);
    // A NaN product (a NaN element; a zero times an infinite S_enc_x, which a scale byte of 0 or a tiny tensor
    // amax produce; anything times a NaN S_enc_x) has code 0 by the reference's rule, not the hardware's: lanes
    // that hold one convert again by the reference's table (a wave-uniform branch that is rarely taken)
    const bool special = any_nan<G>(w);
    if (__builtin_amdgcn_ballot_w64(special) != 0) {
      uint32_t exact = 0;
#pragma unroll
      for (int k = 0; k < G; ++k) exact |= f16_to_f4_exact<G>(h, k) << (4 * k);
      codes = special ? exact : codes;
    }
    if (G == 4) *reinterpret_cast<uint16_t*>(my_codes + (j * 64 + lane) * 2) = uint16_t(codes);
    else *reinterpret_cast<uint32_t*>(my_codes + (j * 64 + lane) * 4) = codes;
    if ((lane & (LPB - 1)) == 0) my_scales[(j * 64 + lane) / LPB] = uint8_t(s8);
  }
  // this wave's own LDS region only: program order suffices, no barrier
  const int64_t left = nvec - span;                    // vectors of this span that exist (>= 1)
  const int64_t code_bytes = (left < kTrips * 64 ? left : kTrips * 64) * kCodeBytes;
  const int64_t scale_bytes = (left < kTrips * 64 ? left : kTrips * 64) / LPB;
  uint8_t* qo = q + span * kCodeBytes;
  uint8_t* so = scales + span / LPB;
#pragma unroll
  for (int c = 0; c < kSpanCodes / 1024; ++c) {
    const int o = (c * 64 + lane) * 16;
    const u32x4 vv = *reinterpret_cast<const u32x4*>(my_codes + o);
    if (o + 16 <= code_bytes) {
      *reinterpret_cast<u32x4*>(qo + o) = vv;            // q is 16-byte aligned (checked by the host side)
    } else {
      for (int b = 0; b < 16; b += 2)                    // ragged end: code bytes come in pairs at least
        if (o + b < code_bytes) *reinterpret_cast<uint16_t*>(qo + o + b) = uint16_t(vv[b >> 2] >> (8 * (b & 3)));
    }
  }
  if (lane * 4 < kSpanScales) {
    const int o = lane * 4;
    const uint32_t vv = *reinterpret_cast<const uint32_t*>(my_scales + o);
    if (o + 4 <= scale_bytes && (reinterpret_cast<uintptr_t>(so) & 3) == 0) {
      *reinterpret_cast<uint32_t*>(so + o) = vv;
    } else {
      for (int b = 0; b < 4; ++b)
        if (o + b < scale_bytes) so[o + b] = uint8_t(vv >> (8 * b));
    }
  }
}

// (q_packed, scales, tensor_amax, y, nvec) ; nvec 128-bit vectors of y
template <typename Y>
__device__ __forceinline__ void dequantize_body(const uint8_t* __restrict__ q, const uint8_t* __restrict__ scales,
                                                const float* __restrict__ tensor_amax, typename Y::storage* __restrict__ y,
                                                int64_t nvec) {
  constexpr int G = FloatGroup<Y>::G;
  constexpr int LPB = 16 / G;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t span = (int64_t(blockIdx.x) * (kThreads / 64) + wave) * (kTrips * 64);
  if (span >= nvec) return;
  const float s_dec = *tensor_amax / 2688.0f;
  uint32_t codes[kTrips], s8[kTrips];
#pragma unroll
  for (int j = 0; j < kTrips; ++j) {
    int64_t v = span + j * 64 + lane;
    v = v < nvec ? v : nvec - 1;
    codes[j] = G == 4 ? uint32_t(*reinterpret_cast<const uint16_t*>(q + v * 2)) : *reinterpret_cast<const uint32_t*>(q + v * 4);
    s8[j] = scales[v / LPB];
  }
#pragma unroll
  for (int j = 0; j < kTrips; ++j) {
    const int64_t v = span + j * 64 + lane;
    const float u = f8_to_f32<0>(s8[j]) * s_dec;
    float out[G];
#pragma unroll
    for (int k = 0; k < G; k += 2) {
      f2 p;
      if (k == 0) p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(codes[j], 1.0f, 0);
      else if (k == 2) p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(codes[j], 1.0f, 1);
      else if (k == 4) p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(codes[j], 1.0f, 2);
      else p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(codes[j], 1.0f, 3);
      out[k] = p[0] * u;
      out[k + 1] = p[1] * u;
    }
    if (v < nvec) FloatGroup<Y>::store(y + v * G, out);
  }
}

// ---- blocks of 16 along the SECOND-TO-LAST axis ([d0, d1] view, d0 % 16 == 0) ----------------------
// A lane owns G neighbouring columns of one block row: 16 vectors, one per row, a row's 64 vectors
// of a wave being 1 KiB of contiguous memory.  The block amax is a maximum down the lane's own
// registers, one chain per column.  Per row a wave stores 64 x G/2 bytes of codes and per block row
// 64 x G scale bytes, each contiguous.
// (x, q_packed, scales, tensor_amax, d0, d1) ; d1 % G == 0 ; one lane per (block row, column group)
template <typename X>
__device__ __forceinline__ void quantize_cols_body(const typename X::storage* __restrict__ x, uint8_t* __restrict__ q,
                                                   uint8_t* __restrict__ scales, const float* __restrict__ tensor_amax,
                                                   int64_t d0, int64_t d1) {
  constexpr int G = FloatGroup<X>::G;
  __shared__ float inverse_scale[256];
  const int64_t groups = d1 / G, units = (d0 / 16) * groups;
  const int64_t u = int64_t(blockIdx.x) * kThreads + threadIdx.x;
  const float s_enc = 2688.0f / *tensor_amax;
  fill_inverse_scales(inverse_scale, s_enc);
  if (u >= units) return;
  const int64_t rb = u / groups, c0 = (u - rb * groups) * G;
  const typename X::storage* xp = x + rb * 16 * d1 + c0;
  u32x4 t[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) t[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xp + r * d1));
  float amax[G];
#pragma unroll
  for (int k = 0; k < G; ++k) amax[k] = 0.0f;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    float v[G];
    FloatGroup<X>::unpack(t[r], v);
#pragma unroll
    for (int k = 0; k < G; ++k) amax[k] = fmaxf(amax[k], fabsf(v[k]));
  }
  float s_enc_x[G];
  uint32_t s8[G];
#pragma unroll
  for (int k = 0; k < G; ++k) {
    const float s_dec_x = divide_by_six(amax[k]);
    uint32_t b = f32x2_to_f8_ieee(s_dec_x * s_enc, 0.0f) & 0xFFu;
    b = (b & 0x7Fu) == 0x7Fu ? 0x7Fu : b;
    s8[k] = b;
    s_enc_x[k] = inverse_scale[b];                     // = s_enc / f32(b), the same IEEE quotient
  }
  uint8_t* sp = scales + rb * d1 + c0;
  if (G == 4) {
    *reinterpret_cast<uint32_t*>(sp) = s8[0] | (s8[1] << 8) | (s8[2] << 16) | (s8[3] << 24);
  } else {
    u32x2 w = {s8[0] | (s8[1] << 8) | (s8[2] << 16) | (s8[3] << 24),
               s8[4 % G] | (s8[5 % G] << 8) | (s8[6 % G] << 16) | (s8[7 % G] << 24)};
    *reinterpret_cast<u32x2*>(sp) = w;
  }
  uint8_t* qp = q + (rb * 16 * d1 + c0) / 2;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    float v[G], w[G];
    FloatGroup<X>::unpack(t[r], v);
#pragma unroll
    for (int k = 0; k < G; ++k) w[k] = v[k] * s_enc_x[k];
    uint32_t h[G / 2];
    products_to_f16<G>(w, h);
    uint32_t codes = f16_to_f4<G>(h);
    const bool special = any_nan<G>(w);                // a NaN product: the reference's table (see quantize_body)
    if (__builtin_amdgcn_ballot_w64(special) != 0) {
      uint32_t exact = 0;
#pragma unroll
      for (int k = 0; k < G; ++k) exact |= f16_to_f4_exact<G>(h, k) << (4 * k);
      codes = special ? exact : codes;
    }
    if (G == 4) *reinterpret_cast<uint16_t*>(qp + r * (d1 / 2)) = uint16_t(codes);
    else *reinterpret_cast<uint32_t*>(qp + r * (d1 / 2)) = codes;
  }
}

// (q_packed, scales, tensor_amax, y, d0, d1) ; one lane per output vector
template <typename Y>
__device__ __forceinline__ void dequantize_cols_body(const uint8_t* __restrict__ q, const uint8_t* __restrict__ scales,
                                                     const float* __restrict__ tensor_amax,
                                                     typename Y::storage* __restrict__ y, int64_t d0, int64_t d1) {
  constexpr int G = FloatGroup<Y>::G;
  const int64_t groups = d1 / G, nvec = d0 * groups;
  const float s_dec = *tensor_amax / 2688.0f;
  const int64_t stride = int64_t(gridDim.x) * kThreads;
  for (int64_t v = int64_t(blockIdx.x) * kThreads + threadIdx.x; v < nvec; v += stride) {
    const int64_t r = v / groups, c0 = (v - r * groups) * G;
    const uint32_t codes = G == 4 ? uint32_t(*reinterpret_cast<const uint16_t*>(q + v * 2)) : *reinterpret_cast<const uint32_t*>(q + v * 4);
    const uint8_t* sp = scales + (r / 16) * d1 + c0;
    uint32_t sw[2];
    sw[0] = *reinterpret_cast<const uint32_t*>(sp);
    sw[1] = G == 8 ? *reinterpret_cast<const uint32_t*>(sp + 4) : 0u;
    float out[G];
#pragma unroll
    for (int k = 0; k < G; k += 2) {
      f2 p;
      if (k == 0) p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(codes, 1.0f, 0);
      else if (k == 2) p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(codes, 1.0f, 1);
      else if (k == 4) p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(codes, 1.0f, 2);
      else p = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(codes, 1.0f, 3);
      const uint32_t word = sw[k / 4];
      const float u0 = ((k & 3) == 0 ? f8_to_f32<0>(word) : f8_to_f32<2>(word)) * s_dec;
      const float u1 = ((k & 3) == 0 ? f8_to_f32<1>(word) : f8_to_f32<3>(word)) * s_dec;
      out[k] = p[0] * u0;
      out[k + 1] = p[1] * u1;
    }
    FloatGroup<Y>::store(y + v * G, out);
  }
}

}  // namespace nvfp4_cluster

// mtrt_nvfp4_q_<t>(x, q_packed, scales, tensor_amax, nvec) ; mtrt_nvfp4_dq_<t>(q_packed, scales, tensor_amax, y, nvec)
// grid = ceil(nvec / (4 waves * 8 trips * 64)), block = 256; x / y and q_packed 16-byte aligned.
#define MTRT_NVFP4_KERNELS(XN, XT)                                                                                      \
  extern "C" __global__ void __launch_bounds__(nvfp4_cluster::kThreads) mtrt_nvfp4_q_##XN(                               \
      const XT::storage* x, uint8_t* q, uint8_t* scales, const float* tensor_amax, int64_t nvec) {                      \
    nvfp4_cluster::quantize_body<XT>(x, q, scales, tensor_amax, nvec);                                                  \
  }                                                                                                                     \
  extern "C" __global__ void __launch_bounds__(nvfp4_cluster::kThreads) mtrt_nvfp4_dq_##XN(                              \
      const uint8_t* q, const uint8_t* scales, const float* tensor_amax, XT::storage* y, int64_t nvec) {                \
    nvfp4_cluster::dequantize_body<XT>(q, scales, tensor_amax, y, nvec);                                                \
  }
// Blocks along the second-to-last axis: mtrt_nvfp4_qc_<t>(x, q_packed, scales, tensor_amax, d0, d1) with
// grid = ceil((d0 / 16) * (d1 / G) / 256); mtrt_nvfp4_dqc_<t>(q_packed, scales, tensor_amax, y, d0, d1).
// d1 % G == 0 (G = 4 for f32, 8 for f16 / bf16), x / y rows 16-byte aligned, scales 4- (G = 4) or 8-byte aligned.
#define MTRT_NVFP4_COL_KERNELS(XN, XT)                                                                                  \
  extern "C" __global__ void __launch_bounds__(nvfp4_cluster::kThreads) mtrt_nvfp4_qc_##XN(                              \
      const XT::storage* x, uint8_t* q, uint8_t* scales, const float* tensor_amax, int64_t d0, int64_t d1) {            \
    nvfp4_cluster::quantize_cols_body<XT>(x, q, scales, tensor_amax, d0, d1);                                           \
  }                                                                                                                     \
  extern "C" __global__ void __launch_bounds__(nvfp4_cluster::kThreads) mtrt_nvfp4_dqc_##XN(                             \
      const uint8_t* q, const uint8_t* scales, const float* tensor_amax, XT::storage* y, int64_t d0, int64_t d1) {      \
    nvfp4_cluster::dequantize_cols_body<XT>(q, scales, tensor_amax, y, d0, d1);                                         \
  }
MTRT_NVFP4_COL_KERNELS(f32, mtrt_dev::F32)
MTRT_NVFP4_COL_KERNELS(f16, mtrt_dev::F16)
MTRT_NVFP4_COL_KERNELS(bf16, mtrt_dev::BF16)
MTRT_NVFP4_KERNELS(f32, mtrt_dev::F32)
MTRT_NVFP4_KERNELS(f16, mtrt_dev::F16)
MTRT_NVFP4_KERNELS(bf16, mtrt_dev::BF16)
