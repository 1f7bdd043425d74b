// TEST INFRASTRUCTURE — CPU oracle, not a product path.  See mtrt_oracle.h.
//
// Straight-loop restatement of the reference host backend's execution of the
// five benchmark programs.  Scalar op semantics follow
//   mlir-tensorrt/executor/lib/Runtime/Backend/Lua/Modules/Core/CoreModule.cpp
//     :473-483  _divf_f32   = `lhs / rhs` on float
//     :72-98, :647-675  _fptosi_f32_i8 = static_cast (exact after the clamp), _fptosi_f32_i4 =
//               Int4(trunc(x)) saturating
//     :791-808  _truncf_f32_{f16,bf16,f8E4M3FN} / _extf = the DataTypes.cpp constructors
//     :1088-1092, :1145-1170  exp / sqrt = libm in f32
//   mlir-tensorrt/executor/lib/Passes/ExpandMathOps.cpp:101-140
//     roundeven -> exact round-half-even; rsqrt -> 1/sqrt; fma -> a*b+c; clampf -> max(min(x,hi),lo)
//   mlir-tensorrt/common/lib/Dialect/LinalgExt/Transforms/ToLoopsOpInterfaceImpl.cpp:142-203
//     one loop per iteration dim in order; reductions accumulate sequentially.
// Build with -ffp-contract=off so no op pair is fused.
#include "mtrt_oracle.h"
#include "lowp.hpp"

#include <cmath>
#include <cstdlib>
#include <vector>

using namespace orc;

namespace {

inline float load_as_f32(const void *p, int dtype, int64_t i) {
  switch (dtype) {
  case ORC_F32:
    return static_cast<const float *>(p)[i];
  case ORC_F16:
    return f16_to_f32(static_cast<const uint16_t *>(p)[i]);
  case ORC_BF16:
    return bf16_to_f32(static_cast<const uint16_t *>(p)[i]);
  case ORC_I8:
    return float(static_cast<const int8_t *>(p)[i]);
  case ORC_F8E4M3FN:
    return f8e4m3fn_to_f32(static_cast<const uint8_t *>(p)[i]);
  case ORC_I4:
    return float(int4_sign_extend(static_cast<const uint8_t *>(p)[i]));
  case ORC_I4_PACKED: {
    const uint8_t byte = static_cast<const uint8_t *>(p)[i >> 1];
    return float(int4_sign_extend((i & 1) ? (byte >> 4) : (byte & 0xF)));
  }
  case ORC_I32:
    return float(static_cast<const int32_t *>(p)[i]);
  case ORC_F4_PACKED: {
    const uint8_t byte = static_cast<const uint8_t *>(p)[i >> 1];
    return f4e2m1fn_to_f32((i & 1) ? (byte >> 4) : (byte & 0xF));
  }
  }
  std::abort();
}

inline void store_float(void *p, int dtype, int64_t i, float v, ConvMode mode) {
  switch (dtype) {
  case ORC_F32:
    static_cast<float *>(p)[i] = v;
    return;
  case ORC_F16:
    static_cast<uint16_t *>(p)[i] = f32_to_f16(v, mode);
    return;
  case ORC_BF16:
    static_cast<uint16_t *>(p)[i] = f32_to_bf16(v, mode);
    return;
  }
  std::abort();
}

inline float round_half_even(float v) { return std::nearbyintf(v); } // default FE_TONEAREST
inline float clampf(float v, float lo, float hi) { return std::fmax(std::fmin(v, hi), lo); }

inline int64_t scale_index(int kind, int64_t r, int64_t c, int64_t d1, int64_t nb) {
  switch (kind) {
  case ORC_SCALE_UNIFORM:
    return 0;
  case ORC_SCALE_ROW:
    return r % nb;
  case ORC_SCALE_COL:
    return (r / nb) * d1 + c;
  }
  std::abort();
}

} // namespace

extern "C" {

uint8_t orc_f32_to_f8e4m3fn(float x, int mode) { return f32_to_f8e4m3fn(x, ConvMode(mode)); }
float orc_f8e4m3fn_to_f32(uint8_t b) { return f8e4m3fn_to_f32(b); }
uint16_t orc_f32_to_f16(float x, int mode) { return f32_to_f16(x, ConvMode(mode)); }
float orc_f16_to_f32(uint16_t b) { return f16_to_f32(b); }
uint16_t orc_f32_to_bf16(float x, int mode) { return f32_to_bf16(x, ConvMode(mode)); }
float orc_bf16_to_f32(uint16_t b) { return bf16_to_f32(b); }
int8_t orc_int4_saturate(int32_t v) { return int4_saturate(v); }
int8_t orc_int4_sign_extend(uint8_t nibble) { return int4_sign_extend(nibble); }

void orc_narrow(const float *src, void *dst, int dst_dtype, int64_t n, int mode) {
  const ConvMode m = ConvMode(mode);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    if (dst_dtype == ORC_F8E4M3FN)
      static_cast<uint8_t *>(dst)[i] = f32_to_f8e4m3fn(src[i], m);
    else
      store_float(dst, dst_dtype, i, src[i], m);
  }
}

void orc_widen(const void *src, int src_dtype, float *dst, int64_t n) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i)
    dst[i] = load_as_f32(src, src_dtype, i);
}

void orc_pack_int4(const int8_t *unpacked, uint8_t *packed, int64_t n) {
  for (int64_t i = 0; i < n; i += 2) {
    const uint8_t lo = uint8_t(unpacked[i]) & 0xF;
    const uint8_t hi = (i + 1 < n) ? (uint8_t(unpacked[i + 1]) & 0xF) : 0;
    packed[i >> 1] = uint8_t(lo | (hi << 4));
  }
}

void orc_unpack_int4(const uint8_t *packed, int8_t *unpacked, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    const uint8_t byte = packed[i >> 1];
    unpacked[i] = int4_sign_extend((i & 1) ? (byte >> 4) : (byte & 0xF));
  }
}

float orc_amax(const void *x, int dtype, int64_t n) {
  float amax = 0.0f; // reduce init for max(abs(.)) is 0 (abs >= 0)
#pragma omp parallel for schedule(static) reduction(max : amax)
  for (int64_t i = 0; i < n; ++i) {
    const float a = std::fabs(load_as_f32(x, dtype, i));
    amax = a > amax ? a : amax;
  }
  return amax;
}

float orc_scale_from_amax(float amax, float qmax) { return amax / qmax; }

void orc_amax_scales(const void *x, int dtype, int scale_kind, int64_t d0, int64_t d1, int64_t nb, float qmax,
                     float *amax_out, float *scale_out) {
  const int64_t count = scale_kind == ORC_SCALE_UNIFORM ? 1 : (scale_kind == ORC_SCALE_ROW ? nb : (d0 / nb) * d1);
  std::vector<float> amax(size_t(count), 0.0f);       // reduce init for max(abs(.)) is 0
  for (int64_t r = 0; r < d0; ++r)
    for (int64_t c = 0; c < d1; ++c) {
      const float a = std::fabs(load_as_f32(x, dtype, r * d1 + c));
      float &m = amax[size_t(scale_index(scale_kind, r, c, d1, nb))];
      m = a > m ? a : m;
    }
  for (int64_t i = 0; i < count; ++i) {
    if (amax_out)
      amax_out[i] = amax[size_t(i)];
    if (scale_out)
      scale_out[i] = amax[size_t(i)] / qmax;
  }
}

void orc_quantize(const void *x, int in_dtype, void *q, int out_dtype, const float *scale,
                  int scale_kind, int64_t d0, int64_t d1, int64_t nb, int flags, int mode) {
  const ConvMode m = ConvMode(mode);
  float lo, hi;
  bool round_int = true;
  switch (out_dtype) {
  case ORC_I8:
    lo = -128.0f, hi = 127.0f;
    break;
  case ORC_F8E4M3FN:
    lo = -448.0f, hi = 448.0f;
    round_int = (flags & ORC_Q_ROUND_TO_INT) != 0;
    break;
  case ORC_I4:
  case ORC_I4_PACKED:
    lo = -8.0f, hi = 7.0f;
    break;
  case ORC_F4_PACKED:
    lo = -6.0f, hi = 6.0f;
    round_int = (flags & ORC_Q_ROUND_TO_INT) != 0;
    break;
  default:
    std::abort();
  }
  // packed codes: a byte holds elements (2j, 2j+1) of the flattened array, so rows of odd length share
  // bytes with their neighbours and must not be handed to different threads
  const bool rows_share_bytes = (out_dtype == ORC_I4_PACKED || out_dtype == ORC_F4_PACKED) && (d1 & 1);
#pragma omp parallel for schedule(static) if (!rows_share_bytes)
  for (int64_t r = 0; r < d0; ++r) {
    for (int64_t c = 0; c < d1; ++c) {
      const int64_t i = r * d1 + c;
      const float s = scale[scale_index(scale_kind, r, c, d1, nb)];
      float v = load_as_f32(x, in_dtype, i) / s;
      if (round_int)
        v = round_half_even(v);
      v = clampf(v, lo, hi);
      switch (out_dtype) {
      case ORC_I8:
        static_cast<int8_t *>(q)[i] = static_cast<int8_t>(v);
        break;
      case ORC_F8E4M3FN:
        if (flags & ORC_F8_VIA_F16)
          v = f16_to_f32(f32_to_f16(v, kIeee));   // first rounding; the widening back is exact
        static_cast<uint8_t *>(q)[i] = f32_to_f8e4m3fn(v, (flags & ORC_F8_VIA_F16) ? kIeee : m);
        break;
      case ORC_I4:
        static_cast<uint8_t *>(q)[i] = uint8_t(int4_saturate(int(std::trunc(v)))) & 0xF;
        break;
      case ORC_I4_PACKED: {
        const uint8_t nib = uint8_t(int4_saturate(int(std::trunc(v)))) & 0xF;
        uint8_t *b = static_cast<uint8_t *>(q) + (i >> 1);
        *b = (i & 1) ? uint8_t((*b & 0x0F) | (nib << 4)) : uint8_t((*b & 0xF0) | nib);
        break;
      }
      case ORC_F4_PACKED: {
        const uint8_t nib = f16_to_f4e2m1fn(f32_to_f16(v, m), m);
        uint8_t *b = static_cast<uint8_t *>(q) + (i >> 1);
        *b = (i & 1) ? uint8_t((*b & 0x0F) | (nib << 4)) : uint8_t((*b & 0xF0) | nib);
        break;
      }
      }
    }
  }
}

void orc_dequantize(const void *q, int in_dtype, void *y, int out_dtype, const float *scale,
                    int scale_kind, int64_t d0, int64_t d1, int64_t nb, int mode) {
  const ConvMode m = ConvMode(mode);
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < d0; ++r)
    for (int64_t c = 0; c < d1; ++c) {
      const int64_t i = r * d1 + c;
      const float s = scale[scale_index(scale_kind, r, c, d1, nb)];
      store_float(y, out_dtype, i, load_as_f32(q, in_dtype, i) * s, m);
    }
}

uint8_t orc_f16_to_f4e2m1fn(uint16_t h, int mode) { return f16_to_f4e2m1fn(h, ConvMode(mode)); }
float orc_f4e2m1fn_to_f32(uint8_t code) { return f4e2m1fn_to_f32(code); }

// block_axis 1: blocks of 16 along the last axis (d1); 0: along the second-to-last axis (d0).
// Scales are laid out like the input with the blocked extent divided by 16.
void orc_nvfp4_quantize(const void *x, int in_dtype, uint8_t *q_packed, uint8_t *scales, float tensor_amax,
                        int64_t d0, int64_t d1, int block_axis, int mode) {
  const ConvMode m = ConvMode(mode);
  const int64_t nb0 = block_axis ? d0 : d0 / 16, nb1 = block_axis ? d1 / 16 : d1;
  const int64_t step = block_axis ? 1 : d1;              // element stride inside a block
  const float s_enc = 2688.0f / tensor_amax;             // 6 * 448 / amax, one f32 divide
#pragma omp parallel for schedule(static)
  for (int64_t b0 = 0; b0 < nb0; ++b0) {
    for (int64_t b1 = 0; b1 < nb1; ++b1) {
      const int64_t base = block_axis ? b0 * d1 + b1 * 16 : b0 * 16 * d1 + b1;
      float amax = 0.0f;
      for (int i = 0; i < 16; ++i)
        amax = std::fmax(amax, std::fabs(load_as_f32(x, in_dtype, base + i * step)));
      const float s_dec_x = amax / 6.0f;
      const uint8_t s8 = f32_to_f8e4m3fn(s_dec_x * s_enc, m);
      scales[b0 * nb1 + b1] = s8;
      const float s_enc_x = s_enc / f8e4m3fn_to_f32(s8);
      for (int i = 0; i < 16; ++i) {
        const int64_t e = base + i * step;
        const float v = load_as_f32(x, in_dtype, e) * s_enc_x;
        const uint8_t c = f16_to_f4e2m1fn(f32_to_f16(v, m), m);
        uint8_t *byte = q_packed + (e >> 1);             // neighbours along d1 share a byte
        if (block_axis) {
          *byte = (e & 1) ? uint8_t((*byte & 0x0F) | (c << 4)) : uint8_t((*byte & 0xF0) | c);
        } else {
#pragma omp critical(nvfp4_nibble)
          *byte = (e & 1) ? uint8_t((*byte & 0x0F) | (c << 4)) : uint8_t((*byte & 0xF0) | c);
        }
      }
    }
  }
}

void orc_nvfp4_dequantize(const uint8_t *q_packed, const uint8_t *scales, float tensor_amax, void *y,
                          int out_dtype, int64_t d0, int64_t d1, int block_axis, int mode) {
  const ConvMode m = ConvMode(mode);
  const int64_t nb1 = block_axis ? d1 / 16 : d1;
  const float s_dec = tensor_amax / 2688.0f;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < d0; ++r) {
    for (int64_t c = 0; c < d1; ++c) {
      const int64_t e = r * d1 + c;
      const int64_t si = block_axis ? r * nb1 + c / 16 : (r / 16) * nb1 + c;
      const float u = f8e4m3fn_to_f32(scales[si]) * s_dec;
      const uint8_t code = (q_packed[e / 2] >> (4 * (e & 1))) & 0xF;
      store_float(y, out_dtype, e, f4e2m1fn_to_f32(code) * u, m);
    }
  }
}

void orc_layernorm(const void *x, const void *gamma, const void *beta, void *y, int dtype,
                   int64_t rows, int64_t d, float eps, int mode) {
  const ConvMode m = ConvMode(mode);
  const float fd = float(d);
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const int64_t base = r * d;
    float sum = 0.0f;
    for (int64_t c = 0; c < d; ++c)
      sum = sum + load_as_f32(x, dtype, base + c);
    const float mu = sum / fd;
    float sq = 0.0f;
    for (int64_t c = 0; c < d; ++c) {
      const float dv = load_as_f32(x, dtype, base + c) - mu;
      sq = sq + dv * dv;
    }
    const float var = sq / fd;
    const float rstd = 1.0f / std::sqrt(var + eps);
    for (int64_t c = 0; c < d; ++c) {
      const float dv = load_as_f32(x, dtype, base + c) - mu;
      const float g = load_as_f32(gamma, dtype, c);
      const float b = load_as_f32(beta, dtype, c);
      store_float(y, dtype, base + c, ((dv * rstd) * g) + b, m);
    }
  }
}

void orc_softmax(const void *x, void *y, int dtype, int64_t rows, int64_t d, int mode) {
  const ConvMode m = ConvMode(mode);
#pragma omp parallel
  {
    std::vector<float> e(static_cast<size_t>(d));
#pragma omp for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
      const int64_t base = r * d;
      float mx = -INFINITY;
      for (int64_t c = 0; c < d; ++c) {
        const float v = load_as_f32(x, dtype, base + c);
        mx = v > mx ? v : mx;
      }
      float s = 0.0f;
      for (int64_t c = 0; c < d; ++c) {
        e[c] = std::exp(load_as_f32(x, dtype, base + c) - mx);
        s = s + e[c];
      }
      for (int64_t c = 0; c < d; ++c)
        store_float(y, dtype, base + c, e[c] / s, m);
    }
  }
}

void orc_gemm_i8_i32(const int8_t *a, const int8_t *w, int32_t *acc, int64_t M, int64_t K,
                     int64_t N) {
#pragma omp parallel for schedule(static)
  for (int64_t mi = 0; mi < M; ++mi) {
    int32_t *row = acc + mi * N;
    for (int64_t n = 0; n < N; ++n)
      row[n] = 0;
    for (int64_t k = 0; k < K; ++k) {
      const int32_t av = a[mi * K + k];
      const int8_t *wr = w + k * N;
      for (int64_t n = 0; n < N; ++n)
        row[n] += av * int32_t(wr[n]);
    }
  }
}

void orc_gemm_w8a8(const int8_t *a, const int8_t *w, const float *a_scale, const float *w_scale,
                   uint16_t *y, int64_t M, int64_t K, int64_t N, int64_t m0, int64_t mcount,
                   int mode) {
  (void)M;
  const ConvMode cm = ConvMode(mode);
#pragma omp parallel
  {
    std::vector<int32_t> row(static_cast<size_t>(N));
#pragma omp for schedule(static)
    for (int64_t mi = m0; mi < m0 + mcount; ++mi) {
      for (int64_t n = 0; n < N; ++n)
        row[n] = 0;
      for (int64_t k = 0; k < K; ++k) {
        const int32_t av = a[mi * K + k];
        const int8_t *wr = w + k * N;
        for (int64_t n = 0; n < N; ++n)
          row[n] += av * int32_t(wr[n]);
      }
      for (int64_t n = 0; n < N; ++n)
        y[mi * N + n] = f32_to_f16((float(row[n]) * a_scale[mi]) * w_scale[n], cm);
    }
  }
}

void orc_gemm_w4a16(const uint16_t *a, const uint8_t *w_packed, const uint16_t *scale, uint16_t *y,
                    int64_t M, int64_t K, int64_t N, int64_t block, int64_t m0, int64_t mcount,
                    int mode) {
  (void)M;
  const ConvMode cm = ConvMode(mode);
  // wd[k,n] = f16(f16(w) * s): the f32 product of an int4 and an f16 is exact, so one
  // rounding to f16 equals the f16 multiply the program states.
  std::vector<float> wd(static_cast<size_t>(K) * size_t(N));
#pragma omp parallel for schedule(static)
  for (int64_t k = 0; k < K; ++k)
    for (int64_t n = 0; n < N; ++n) {
      const int64_t i = k * N + n;
      const uint8_t byte = w_packed[i >> 1];
      const float wv = float(int4_sign_extend((i & 1) ? (byte >> 4) : (byte & 0xF)));
      const float sv = f16_to_f32(scale[(k / block) * N + n]);
      wd[size_t(i)] = f16_to_f32(f32_to_f16(wv * sv, cm));
    }
#pragma omp parallel
  {
    std::vector<float> row(static_cast<size_t>(N));
#pragma omp for schedule(static)
    for (int64_t mi = m0; mi < m0 + mcount; ++mi) {
      for (int64_t n = 0; n < N; ++n)
        row[n] = 0.0f;
      for (int64_t k = 0; k < K; ++k) {
        const float av = f16_to_f32(a[mi * K + k]);
        const float *wr = wd.data() + size_t(k) * size_t(N);
        for (int64_t n = 0; n < N; ++n)
          row[n] = row[n] + av * wr[n];
      }
      for (int64_t n = 0; n < N; ++n)
        y[mi * N + n] = f32_to_f16(row[n], cm);
    }
  }
}

} // extern "C"
