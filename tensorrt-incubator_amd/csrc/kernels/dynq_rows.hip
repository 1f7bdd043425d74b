// Dynamic per-row (per-token) quantization in ONE launch:
//     amax[r]  = max_c |f32(x[r,c])|
//     scale[r] = amax[r] / qmax                                   (one IEEE divide)
//     q[r,c]   = convert(clamp(lo, [rne](f32(x[r,c]) / scale[r]), hi))
// i.e. the {abs, reduce-max} cluster of a row, the scale rule of the calibration flow
// (tripy/examples/nanogpt/weight_loader.py:67-68, 102-115) and the quantize cluster
// (mlir-tensorrt/compiler/lib/Dialect/StablehloExt/Transforms/StablehloRaiseQDQ.cpp:233-265) fused the way the
// reference's segmentation pulls single-use elementwise producers into their consumer
// (mlir-tensorrt/compiler/lib/Backends/Kernel/KernelSegmentation.cpp:84-100).  This is what produces the int8
// activations and the per-token scales a_scale[m] of the W8A8 GEMM.
//
// The two-launch form (amax per row, then quantize with row scales) reads the activations twice.  Here the row
// stays in registers between the reduction and the quantization: a wave owns a row (NV <= 8 128-bit vectors per lane,
// up to 64 * NV vectors per row) or, for longer rows, the four waves of a workgroup share one and meet in LDS;
// the row maximum is a cross-lane exchange, the quotient the short exact division of qdq.hip (ExactDivisor), so
// codes and scales are bit-identical to the two launches.  Loads are unconditional (lanes past the end of the row
// repeat its last vector, which cannot change a maximum) and only the stores are predicated.
#include "common.hpp"

namespace dynq_rows_cluster {

using namespace mtrt_dev;
using namespace amax_cluster;
using namespace qdq_cluster;

// WAVES waves per row (1: a wave per row, kWavesPerBlock rows per workgroup; 4: the workgroup's four waves share a row)
constexpr int kThreads = 256;

template <typename X, typename Q, int NV, int WAVES>
__device__ __forceinline__ void body(const typename X::storage* __restrict__ x, typename Q::storage* __restrict__ q, int64_t rows,
                                     int64_t d, float qmax, float* __restrict__ amax_out, float* __restrict__ scale_out, int flags) {
  using FG = FloatGroup<X>;
  using A = AbsBits<X>;
  constexpr int G = FG::G;
  constexpr int kLanes = kWave * WAVES;                // lanes that share a row
  __shared__ uint32_t part[kThreads / kWave];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t row = WAVES == 1 ? int64_t(blockIdx.x) * (kThreads / kWave) + wave : int64_t(blockIdx.x);
  const bool have_row = row < rows;                    // uniform per wave; with WAVES == 4 per workgroup
  const int64_t r = have_row ? row : rows - 1;         // surplus waves of the last workgroup repeat the last row, store nothing
  const uint32_t nvec = uint32_t(d / G);
  const uint32_t first = WAVES == 1 ? uint32_t(lane) : uint32_t(threadIdx.x);
  const typename X::storage* xr = x + r * d;

  u32x4 xin[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const uint32_t v = first + uint32_t(i) * kLanes;
    xin[i] = FG::load(xr + int64_t(v < nvec ? v : nvec - 1) * G);
  }
  uint32_t m = 0;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const uint32_t a = A::of(xin[i]);
    m = m > a ? m : a;
  }
  m = wave_reduce(m, MaxU32());
  if (WAVES > 1) {
    if (lane == 0) part[wave] = m;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < WAVES; ++w) m = m > part[w] ? m : part[w];
  }
  const float amax = A::finish(m);
  const float scale = amax / qmax;                     // one IEEE divide, as the host computes it
  if (have_row && first == 0) {
    if (amax_out) amax_out[row] = amax;
    scale_out[row] = scale;
  }
  const ExactDivisor dv(scale);
  typename Q::storage* qr = q + r * d;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const uint32_t v = first + uint32_t(i) * kLanes;
    float f[G];
    FG::unpack(xin[i], f);
    quantize_group<Q>(dv, f, flags);
    if (have_row && v < nvec) CodeGroup<Q, G>::store(qr, int64_t(v) * G, f, flags);
  }
}

}  // namespace dynq_rows_cluster

// (x [rows, d], q [rows, d], rows, d, qmax, amax_out [rows] or null, scale_out [rows], flags)
//   d % G == 0 (G = 4 for f32, 8 for f16 / bf16), 0 < d / G <= 64 * NV (`_v`) or 256 * NV (`_g4v`), x 16-byte aligned,
//   q aligned to G codes; grid = ceil(rows / 4) (`_v`: a wave per row) or rows (`_g4v`: a workgroup per row), block = 256.
// A wave holds up to 8 vectors per lane (more rows per compute unit in flight than with 16), the workgroup form 4 to 16.
// The 16-vector form of the 16-bit -> f8 pairs needs scratch memory (the host does not launch it: a kernel with more
// than a little scratch pays about 10 us per launch for its allocation) and is not built.
#define MTRT_DYNQ_ROWS_WAVE(XN, XT, QN, QT, NV)                                                                          \
  extern "C" __global__ void __launch_bounds__(256) mtrt_dynq_rows_##XN##_##QN##_v##NV(                                   \
      const XT::storage* x, QT::storage* q, int64_t rows, int64_t d, float qmax, float* amax_out, float* scale_out,       \
      int32_t flags) {                                                                                                    \
    dynq_rows_cluster::body<XT, QT, NV, 1>(x, q, rows, d, qmax, amax_out, scale_out, flags); }
#define MTRT_DYNQ_ROWS_GROUP(XN, XT, QN, QT, NV)                                                                         \
  extern "C" __global__ void __launch_bounds__(256) mtrt_dynq_rows_##XN##_##QN##_g4v##NV(                                 \
      const XT::storage* x, QT::storage* q, int64_t rows, int64_t d, float qmax, float* amax_out, float* scale_out,       \
      int32_t flags) {                                                                                                    \
    dynq_rows_cluster::body<XT, QT, NV, 4>(x, q, rows, d, qmax, amax_out, scale_out, flags); }
#define MTRT_DYNQ_ROWS_KERNELS(XN, XT, QN, QT)                                                                            \
  MTRT_DYNQ_ROWS_WAVE(XN, XT, QN, QT, 1) MTRT_DYNQ_ROWS_WAVE(XN, XT, QN, QT, 2) MTRT_DYNQ_ROWS_WAVE(XN, XT, QN, QT, 4)     \
  MTRT_DYNQ_ROWS_WAVE(XN, XT, QN, QT, 8) MTRT_DYNQ_ROWS_GROUP(XN, XT, QN, QT, 1) MTRT_DYNQ_ROWS_GROUP(XN, XT, QN, QT, 2)  \
  MTRT_DYNQ_ROWS_GROUP(XN, XT, QN, QT, 4) MTRT_DYNQ_ROWS_GROUP(XN, XT, QN, QT, 8)
MTRT_DYNQ_ROWS_KERNELS(f32, F32, i8, I8)
MTRT_DYNQ_ROWS_KERNELS(f32, F32, f8, F8)
MTRT_DYNQ_ROWS_KERNELS(f16, F16, i8, I8)
MTRT_DYNQ_ROWS_KERNELS(f16, F16, f8, F8)
MTRT_DYNQ_ROWS_KERNELS(bf16, BF16, i8, I8)
MTRT_DYNQ_ROWS_KERNELS(bf16, BF16, f8, F8)
MTRT_DYNQ_ROWS_GROUP(f32, F32, i8, I8, 16)
MTRT_DYNQ_ROWS_GROUP(f32, F32, f8, F8, 16)
MTRT_DYNQ_ROWS_GROUP(f16, F16, i8, I8, 16)
MTRT_DYNQ_ROWS_GROUP(bf16, BF16, i8, I8, 16)
