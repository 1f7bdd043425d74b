// Dynamic per-tensor quantization in ONE launch: amax, scale, quantize and dequantize.
//
//   amax = reduce_max(abs(f32(x)));  scale = amax / qmax
//   q = convert(clamp(lo, [rne](f32(x) / scale), hi));  y = narrow(f32(q) * scale)
//
// i.e. the three clusters the kernel backend forms for a dynamic-scale quantization ({abs, reduce-max},
// {divide, round, clamp, convert}, {convert, multiply}: mlir-tensorrt/compiler/lib/Backends/Kernel/
// KernelSegmentation.cpp:53-113; program form StablehloRaiseQDQ.cpp:233-265, 407-418; scale rule
// tripy/examples/nanogpt/weight_loader.py:67-68) run as one kernel for tensors small enough that the whole
// tensor fits in the registers of one grid: x is read once (the two-launch form reads it twice) and the time of
// a second launch is saved, which is most of the cost of a tensor of a few MB.
//
// Shape: gridDim.x workgroups of 1024 lanes, one per compute unit at most; each lane keeps NV 128-bit vectors of
// x in registers.  The workgroups meet in the arrival tree of amax.hip; whoever arrives last at the root
// publishes the maximum (tag in the high half of a 64-bit word), in kCopies copies on cache lines of their own so
// that the polls of the waiting workgroups spread over as many memory-side queues (every device-scope atomic on
// one line is served one after the other; a flat exchange where all workgroups add to and poll one counter was
// measured 5 us slower on 256 workgroups).  Every workgroup needs that word before it can quantize.
// Nothing guarantees that all workgroups of a launch are resident at once (another stream may hold compute
// units), so the wait is BOUNDED: lane 0 polls `spin_limit` times; a workgroup that gives up computes the maximum
// of the whole tensor by itself (slow, same bits) and goes on, which frees its compute unit for the workgroups
// still queued.  No workgroup ever depends on another one making progress.
// The scratch block restores itself: after reading (or giving up on) the result every workgroup arrives at a
// second counter, and the last of them clears the result words and the counter.
//
// scratch (the stream's reduction block, zero on entry and on exit): lines 0..32 arrival tree, lines 33..48 the
// copies of the result word {tag, max bits}, line 49 the second counter.
#include "common.hpp"

namespace dynq_cluster {

using namespace mtrt_dev;
using namespace qdq_cluster;
using namespace amax_cluster;

constexpr int kDynThreads = 1024;
constexpr uint32_t kResultLine = 33, kCopies = 16, kDoneLine = kResultLine + kCopies;

__device__ __forceinline__ uint32_t block_max(uint32_t m, uint32_t* wave_max) {
  m = wave_reduce(m, MaxU32());
  const int wave = threadIdx.x / kWave;
  __syncthreads();                                   // wave_max may still be read from an earlier use
  if ((threadIdx.x & (kWave - 1)) == 0) wave_max[wave] = m;
  __syncthreads();
  uint32_t r = wave_max[0];
#pragma unroll
  for (int w = 1; w < kDynThreads / kWave; ++w) r = r > wave_max[w] ? r : wave_max[w];
  return r;                                          // every lane has the workgroup's maximum
}

template <typename X, typename Q, int NV>
__device__ __forceinline__ void dynqdq_body(const typename X::storage* __restrict__ x, typename Q::storage* __restrict__ q,
                                            typename X::storage* __restrict__ y, int64_t n, float qmax,
                                            float* __restrict__ amax_out, float* __restrict__ scale_out,
                                            uint32_t* __restrict__ scratch, int flags, int spin_limit) {
  using FG = FloatGroup<X>;
  using A = AbsBits<X>;
  constexpr int G = FG::G;
  __shared__ uint32_t wave_max[kDynThreads / kWave];
  __shared__ uint32_t bcast[2];
  const int64_t nvec = n / G;                        // host: n % G == 0, x / y 16-byte aligned
  const int64_t base = int64_t(blockIdx.x) * (kDynThreads * NV) + threadIdx.x;

  u32x4 xin[NV];
  uint32_t m = 0;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int64_t v = base + int64_t(i) * kDynThreads;
    xin[i] = (u32x4){0u, 0u, 0u, 0u};
    if (v < nvec) {
      xin[i] = FG::load(x + v * G);
      const uint32_t a = A::of(xin[i]);
      m = m > a ? m : a;
    }
  }
  m = block_max(m, wave_max);

  unsigned long long* result = reinterpret_cast<unsigned long long*>(scratch + kAmaxLineWords * kResultLine);
  unsigned long long* done = reinterpret_cast<unsigned long long*>(scratch + kAmaxLineWords * kDoneLine);
  constexpr int kLineQwords = kAmaxLineWords / 2;
  if (threadIdx.x == 0) {
    const uint32_t groups = gridDim.x < kAmaxFanIn ? gridDim.x : kAmaxFanIn;
    const uint32_t g = blockIdx.x % groups;
    const uint32_t members = (gridDim.x - g + groups - 1) / groups;
    uint32_t total = m;
    bool have = false;
    if (arrive(scratch + kAmaxLineWords * (1 + g), members, total) && arrive(scratch, groups, total)) {
      // last arrival of the whole grid: publish for the others (tag 1 in the high half)
#pragma unroll
      for (uint32_t c = 0; c < kCopies; ++c)
        __hip_atomic_exchange(result + c * kLineQwords, (1ull << 32) | total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      have = true;
    } else {
      const unsigned long long* mine = result + (blockIdx.x % kCopies) * kLineQwords;
      for (int spin = 0; spin < spin_limit; ++spin) {
        const unsigned long long w = __hip_atomic_load(mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (w >> 32) {
          total = uint32_t(w);
          have = true;
          break;
        }
        __builtin_amdgcn_s_sleep(1);
      }
    }
    bcast[0] = have ? 1u : 0u;
    bcast[1] = total;
  }
  __syncthreads();
  uint32_t total = bcast[1];
  if (bcast[0] == 0u) {
    // gave up waiting: this workgroup reduces the whole tensor itself (max is exact in any order: same bits)
    uint32_t mm = 0;
    for (int64_t v = threadIdx.x; v < nvec; v += kDynThreads) {
      const uint32_t a = A::of(FG::load(x + v * G));
      mm = mm > a ? mm : a;
    }
    total = block_max(mm, wave_max);
  }
  if (threadIdx.x == 0) {
    // second arrival: once every workgroup has the maximum (or has given up) the block returns to zero
    const unsigned long long old = __hip_atomic_fetch_add(done, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (uint32_t(old) == gridDim.x - 1) {
#pragma unroll
      for (uint32_t c = 0; c < kCopies; ++c)
        __hip_atomic_exchange(result + c * kLineQwords, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_exchange(done, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }

  const float amax = A::finish(total);
  const float scale = amax / qmax;                   // one IEEE divide, as the host does it; identical in every workgroup
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    if (amax_out) *amax_out = amax;
    if (scale_out) *scale_out = scale;
  }
  const ExactDivisor dv(scale);
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int64_t v = base + int64_t(i) * kDynThreads;
    if (v < nvec) {
      float f[G];
      FG::unpack(xin[i], f);
#pragma unroll
      for (int k = 0; k < G; ++k) f[k] = finish_quotient<Q>(dv.divide(f[k]), flags);
      CodeGroup<Q, G>::store(q, v * G, f, flags);     // leaves f32(code) in f
      if (y) {
#pragma unroll
        for (int k = 0; k < G; ++k) f[k] = f[k] * scale;
        FG::store(y + v * G, f);
      }
    }
  }
}

}  // namespace dynq_cluster

// (x, q, y or null, n, qmax, amax_out or null, scale_out or null, scratch, flags, spin_limit)
//   n % G == 0 (G = 4 for f32, 8 for f16 / bf16), x and y 16-byte aligned, q aligned to G codes,
//   gridDim.x = ceil(n / G / (1024 * NV)) <= number of compute units, block = 1024.
#define MTRT_DYNQ_KERNEL(XN, XT, QN, QT, NV)                                                                          \
  extern "C" __global__ void __launch_bounds__(1024) mtrt_dynqdq_##XN##_##QN##_v##NV(                                  \
      const XT::storage* x, QT::storage* q, XT::storage* y, int64_t n, float qmax, float* amax_out, float* scale_out,  \
      uint32_t* scratch, int32_t flags, int32_t spin_limit) {                                                          \
    dynq_cluster::dynqdq_body<XT, QT, NV>(x, q, y, n, qmax, amax_out, scale_out, scratch, flags, spin_limit); }
#define MTRT_DYNQ_KERNELS(XN, XT, QN, QT) MTRT_DYNQ_KERNEL(XN, XT, QN, QT, 4) MTRT_DYNQ_KERNEL(XN, XT, QN, QT, 16)
MTRT_DYNQ_KERNELS(f32, F32, i8, I8)
MTRT_DYNQ_KERNELS(f32, F32, f8, F8)
MTRT_DYNQ_KERNELS(f16, F16, i8, I8)
MTRT_DYNQ_KERNELS(f16, F16, f8, F8)
MTRT_DYNQ_KERNELS(bf16, BF16, i8, I8)
MTRT_DYNQ_KERNELS(bf16, BF16, f8, F8)
