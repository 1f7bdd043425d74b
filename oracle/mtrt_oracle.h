/* TEST INFRASTRUCTURE — CPU oracle for the quantization / generated-kernel hot
 * path.  Only tests, the smoke check and the benchmark's cpu_baseline leg may
 * link or load this; the product library never does.
 *
 * Each function restates, as straight loops, what the reference's HOST backend
 * computes for the corresponding StableHLO program: one scalar op per element
 * per step, every f32 op correctly rounded, reductions accumulated sequentially
 * in index order (mlir-tensorrt/common/lib/Dialect/LinalgExt/Transforms/
 * ToLoopsOpInterfaceImpl.cpp:142-203), narrow-type stores through the
 * conversions in lowp.hpp.
 *
 * Parity status of what is NOT pinned by a reference artefact:
 *   - the StableHLO->linalg scalar mappings (divide, round_nearest_even, clamp,
 *     convert) come from openxla/stablehlo @4c0d4841519aed22e3689c30b72a0e4228051249,
 *     which is not in the reference tree: "parity unpinned" for the mapping
 *     itself; the arithmetic they denote (IEEE f32 divide, exact RNE, min/max,
 *     exact int cast after clamp) is pinned by closed forms in the tests.
 *   - last-ulp f32 results of the Lua interpreter (it carries f32 + - * in
 *     double): "parity unpinned"; covered by the 1e-3 float tolerance.
 */
#ifndef MTRT_ORACLE_H
#define MTRT_ORACLE_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types (same numbering as the product header's mtrt_hip_dtype) */
enum {
  ORC_F32 = 0,
  ORC_F16 = 1,
  ORC_BF16 = 2,
  ORC_I8 = 3,
  ORC_F8E4M3FN = 4,
  ORC_I4 = 5,        /* one int4 per byte, low nibble (host / executor storage) */
  ORC_I4_PACKED = 6, /* two per byte, element 2i in the low nibble (TensorRT storage) */
  ORC_I32 = 7,
  ORC_F4_PACKED = 8  /* f4E2M1FN, two per byte, element 2i in the low nibble */
};

/* conversion behaviour, see lowp.hpp */
enum { ORC_IEEE = 0, ORC_REFHOST = 1 };

/* scale addressing for quantize / dequantize; the data tensor is viewed as
 * [d0, d1] row-major (per-channel on a middle axis folds outer*C into d0). */
enum {
  ORC_SCALE_UNIFORM = 0, /* per-tensor: scale[0]                                  */
  ORC_SCALE_ROW = 1,     /* scale[row % nscale]: per-channel on a non-last axis,
                            or blocks along the last axis (d1 = block)           */
  ORC_SCALE_COL = 2      /* scale[(row / block) * d1 + col]: per-channel on the
                            last axis (block = d0) or blocks along axis 0        */
};

/* flags */
enum {
  ORC_Q_ROUND_TO_INT = 1, /* apply round_nearest_even before the clamp (always on
                             for integer targets; optional for f8)                */
  ORC_F8_VIA_F16 = 4      /* f8 target: f32 -> f16 -> f8, each step RNE (IEEE mode of lowp.hpp): the chain
                             the reference's GPU code generator emits
                             (mlir-tensorrt/kernel/lib/Kernel/Transforms/NormalizeQuantizedConversions.cpp:38-118).
                             Pinned as the composition of two pinned conversions: numpy's float16 cast and the
                             golden f16 -> f8 table minted from the reference build agree with it on every
                             witness and random input of tests/test_oracle_programs.py. */
};

/* scalar conversions */
uint8_t orc_f32_to_f8e4m3fn(float x, int mode);
float orc_f8e4m3fn_to_f32(uint8_t b);
uint16_t orc_f32_to_f16(float x, int mode);
float orc_f16_to_f32(uint16_t b);
uint16_t orc_f32_to_bf16(float x, int mode);
float orc_bf16_to_f32(uint16_t b);
int8_t orc_int4_saturate(int32_t v);
int8_t orc_int4_sign_extend(uint8_t nibble);

/* bulk conversions f32 <-> {f16,bf16,f8}; n elements */
void orc_narrow(const float *src, void *dst, int dst_dtype, int64_t n, int mode);
void orc_widen(const void *src, int src_dtype, float *dst, int64_t n);
/* int4 nibble packing: element 2i -> low nibble, 2i+1 -> high nibble
 * (mlir-tensorrt/tensorrt/lib/Target/TensorRTEncodingOpInterface/NetworkEncoder.cpp:552-595) */
void orc_pack_int4(const int8_t *unpacked, uint8_t *packed, int64_t n);
void orc_unpack_int4(const uint8_t *packed, int8_t *unpacked, int64_t n);

/* amax = reduce_max(abs(f32(x))), sequential */
float orc_amax(const void *x, int dtype, int64_t n);
/* scale = amax / qmax, one f32 divide */
float orc_scale_from_amax(float amax, float qmax);

/* amax and scale = amax / qmax for EVERY scale element of the addressing (scale_kind, nscale_or_block) over the
 * [d0, d1] view: the per-channel / block-wise form of the calibration rule
 * (tripy/examples/nanogpt/weight_loader.py:67-68, 102-115).  Outputs: nscale (row kind) or (d0 / block) * d1
 * (col kind) values, 1 for uniform; either may be NULL.  Scale elements no input addresses get amax 0. */
void orc_amax_scales(const void *x, int dtype, int scale_kind, int64_t d0, int64_t d1, int64_t nscale_or_block,
                     float qmax, float *amax_out, float *scale_out);

/* q = convert(clamp(lo, [rne](f32(x) / scale), hi))
 *   (StablehloRaiseQDQ.cpp:233-265; TensorRTOps.td:3133-3194)
 * lo/hi follow out_dtype: i8 [-128,127], f8 [-448,448], i4 [-8,7], f4 [-6,6] (converted through f16). */
void orc_quantize(const void *x, int in_dtype, void *q, int out_dtype, const float *scale,
                  int scale_kind, int64_t d0, int64_t d1, int64_t nscale_or_block, int flags,
                  int mode);
/* y = narrow(f32(q) * scale)  (StablehloRaiseQDQ.cpp:407-418; TensorRTOps.td:3408-3445) */
void orc_dequantize(const void *q, int in_dtype, void *y, int out_dtype, const float *scale,
                    int scale_kind, int64_t d0, int64_t d1, int64_t nscale_or_block, int mode);

/* f4E2M1FN <-> f16/f32 scalar conversions (mlir-tensorrt/executor/lib/Passes/ExpandOps.cpp:365-694) */
uint8_t orc_f16_to_f4e2m1fn(uint16_t h, int mode);
float orc_f4e2m1fn_to_f32(uint8_t code);

/* NVFP4 quantize / dequantize over blocks of 16 along the last axis, as the program of
 * mlir-tensorrt/integrations/PJRT/test/JAX/test_q_dq_nvfp4.py:21-45 (the two-level scaling of
 * tensorrt.dynamic_quantize, TensorRTOps.td:3279-3358), every op in f32:
 *   S_dec_x = max|x_block| / 6 ; S_enc = 2688 / tensor_amax ; s8 = f8e4m3fn(S_dec_x * S_enc)
 *   S_enc_x = S_enc / f32(s8)  ; q = f4e2m1fn(f16(x * S_enc_x))
 *   y = narrow(f32(q) * (f32(s8) * (tensor_amax / 2688)))
 * x: [d0, d1] of in_dtype; block_axis 1: blocks along d1 (d1 % 16 == 0), scales [d0, d1/16];
 * block_axis 0: blocks along d0 (d0 % 16 == 0), scales [d0/16, d1] (the op's two axis choices,
 * mlir-tensorrt/tensorrt/lib/TensorRT/IR/Verification.cpp:1279-1283); q: two codes per byte over the
 * flattened array, element 2i in the low nibble; scales are f8e4m3fn bytes.  Conversions to f4 go through f16 (the only f4 truncation the
 * reference defines).  TensorRT's own IDynamicQuantize arithmetic is closed: "parity unpinned"
 * against it; pinned here are the conversions and the op order of the JAX program. */
void orc_nvfp4_quantize(const void *x, int in_dtype, uint8_t *q_packed, uint8_t *scales, float tensor_amax,
                        int64_t d0, int64_t d1, int block_axis, int mode);
void orc_nvfp4_dequantize(const uint8_t *q_packed, const uint8_t *scales, float tensor_amax, void *y,
                          int out_dtype, int64_t d0, int64_t d1, int block_axis, int mode);

/* LayerNorm over the last dim (RaiseNormalizations.pdll:277-308):
 * mu = sum(xf)/D; d = xf-mu; var = sum(d*d)/D; y = narrow(d * (1/sqrt(var+eps)) * gamma + beta) */
void orc_layernorm(const void *x, const void *gamma, const void *beta, void *y, int dtype,
                   int64_t rows, int64_t d, float eps, int mode);
/* softmax over the last dim (StablehloMatchers.cpp:311-335):
 * m = max; e = exp(xf-m); s = sum(e); y = narrow(e / s) */
void orc_softmax(const void *x, void *y, int dtype, int64_t rows, int64_t d, int mode);

/* acc[m,n] = sum_k i32(a[m,k]) * i32(w[k,n]); a row-major [M,K], w row-major [K,N] */
void orc_gemm_i8_i32(const int8_t *a, const int8_t *w, int32_t *acc, int64_t M, int64_t K,
                     int64_t N);
/* y[m,n] = f16((f32(acc) * a_scale[m]) * w_scale[n]) ; rows [m0, m0+mcount) only */
void orc_gemm_w8a8(const int8_t *a, const int8_t *w, const float *a_scale, const float *w_scale,
                   uint16_t *y_f16, int64_t M, int64_t K, int64_t N, int64_t m0, int64_t mcount,
                   int mode);
/* W4A16: wd = f16(f16(w) * s[k / block, n]); y = f16(sum_k f32(a) * f32(wd)), f32 sequential in k.
 * w packed 2/byte over the flattened [K,N] array; scale f16 [K/block, N]; rows [m0, m0+mcount) */
void orc_gemm_w4a16(const uint16_t *a_f16, const uint8_t *w_packed, const uint16_t *scale_f16,
                    uint16_t *y_f16, int64_t M, int64_t K, int64_t N, int64_t block, int64_t m0,
                    int64_t mcount, int mode);

#ifdef __cplusplus
}
#endif
#endif
