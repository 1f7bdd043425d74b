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
// Shape: gridDim.x workgroups of 1024 lanes, one per compute unit at most (and at most 256); each lane keeps NV
// 128-bit vectors of x in registers.  Every workgroup needs the maximum of all before it can quantize, and the
// exchange is what a launch of a few MB spends most of its time on, so it is built from the cheapest operations
// the memory system has: every workgroup STORES its maximum, tagged with the launch's number, into a slot of its
// own (one device-scope store, nobody waits for it) and then reads all slots (64 lanes x 4 slots, one round trip)
// until every slot carries the tag.  No read-modify-write is on the path: device-scope atomics on one line are
// served one after the other (an arrival tree cost five dependent trips to memory, about 0.9 us each; a single
// counter that all 256 workgroups add to and poll was slower still), plain stores and loads are not.
// The tag is a counter in the scratch block which the workgroups advance when they are done with the slots (a
// maximum that nobody waits for), so the slots never have to be cleared: what an earlier launch left carries an
// older tag.
// Nothing guarantees that all workgroups of a launch are resident at once (another stream may hold compute
// units), so the wait is BOUNDED: `spin_limit` rounds of reads; a workgroup that gives up computes the maximum
// of the whole tensor by itself (slow, same bits) and goes on, which frees its compute unit for the workgroups
// still queued.  No workgroup ever depends on another one making progress.
//
// scratch (the stream's reduction block, zero when the stream first uses it): lines 0..32 belong to the arrival
// tree of amax.hip and are not touched here; lines 33..48 hold the 256 slots {tag, max bits}, line 49 the tag
// counter.  Tags repeat after 2^32 launches.
#include "common.hpp"

namespace dynq_cluster {

using namespace mtrt_dev;
using namespace qdq_cluster;
using namespace amax_cluster;

constexpr int kDynThreads = 1024;
constexpr uint32_t kSlotLine = 33, kSlots = 256, kTagLine = 49;

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

  unsigned long long* slots = reinterpret_cast<unsigned long long*>(scratch + kAmaxLineWords * kSlotLine);
  uint32_t* tag_word = scratch + kAmaxLineWords * kTagLine;
  // asked for before the data, needed after it
  const uint32_t tag = __hip_atomic_load(tag_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;

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

  if (threadIdx.x < kWave) {                         // wave 0: publish, then watch the other slots
    const uint32_t lane = threadIdx.x;
    if (lane == 0)
      __hip_atomic_store(slots + blockIdx.x, ((unsigned long long)tag << 32) | m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    uint32_t total = m, have = 0;
    for (int spin = 0; spin < spin_limit; ++spin) {
      uint32_t mx = m;
      bool ok = true;
#pragma unroll
      for (uint32_t c = 0; c < kSlots / kWave; ++c) {
        const uint32_t idx = lane + kWave * c;
        if (idx < gridDim.x && idx != blockIdx.x) {  // the own slot is known without reading it back
          const unsigned long long w = __hip_atomic_load(slots + idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          ok = ok && uint32_t(w >> 32) == tag;
          mx = mx > uint32_t(w) ? mx : uint32_t(w);
        }
      }
      if (__ballot(ok) == __ballot(true)) {
        total = wave_reduce(mx, MaxU32());
        have = 1;
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
    if (lane == 0) {
      bcast[0] = have;
      bcast[1] = total;
    }
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
  // Done with the slots: advance the tag counter for the next launch on this stream.  Every workgroup does it
  // (a maximum, so it is idempotent) and none waits for an answer: 256 workgroups updating one line within a
  // microsecond take the memory side up to 3 us to serve, and a lane that waited for its turn would hold its
  // whole wave back.  The counter cannot move while a workgroup of this launch has yet to read it: nobody gets
  // here before every slot carries the tag, and a workgroup publishes after it has read the counter.  (Unless
  // somebody gave up waiting: a workgroup that starts after that reads the advanced counter, finds no slot with
  // its tag, gives up in turn and computes the maximum itself; right, only slow, like every give-up.)
  if (threadIdx.x == 0) __hip_atomic_fetch_max(tag_word, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

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
      quantize_group<Q>(dv, f, flags);
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
//   gridDim.x = ceil(n / G / (1024 * NV)) <= min(number of compute units, 256), block = 1024.
#define MTRT_DYNQ_KERNEL(XN, XT, QN, QT, NV)                                                                          \
  extern "C" __global__ void __launch_bounds__(1024) mtrt_dynqdq_##XN##_##QN##_v##NV(                                  \
      const XT::storage* x, QT::storage* q, XT::storage* y, int64_t n, float qmax, float* amax_out, float* scale_out,  \
      uint32_t* scratch, int32_t flags, int32_t spin_limit) {                                                          \
    dynq_cluster::dynqdq_body<XT, QT, NV>(x, q, y, n, qmax, amax_out, scale_out, scratch, flags, spin_limit); }
#define MTRT_DYNQ_KERNELS(XN, XT, QN, QT) MTRT_DYNQ_KERNEL(XN, XT, QN, QT, 4) MTRT_DYNQ_KERNEL(XN, XT, QN, QT, 16)
MTRT_DYNQ_KERNELS(f32, F32, i8, I8)
MTRT_DYNQ_KERNELS(f32, F32, f8, F8)
MTRT_DYNQ_KERNELS(f16, F16, i8, I8)
MTRT_DYNQ_KERNELS(bf16, BF16, i8, I8)
// 16-bit -> f8: four vectors per lane only.  With sixteen the 128 registers a lane of a 1024-lane workgroup has do not
// hold the chunk and part of it goes to scratch memory, whose allocation costs a launch some 10 us (measured: f16
// [32 Mi] to f8 55.8 us against 35.5 us to int8); such tensors take the two launches instead.
MTRT_DYNQ_KERNEL(f16, F16, f8, F8, 4)
MTRT_DYNQ_KERNEL(bf16, BF16, f8, F8, 4)
