// amax cluster: amax = reduce_max(abs(f32(x))) over the whole tensor, plus the
// host-sized follow-up op scale = amax / qmax folded into the same launch.
//
// Reference program: the {abs, reduce-max} codegen cluster that the kernel backend
// forms for a dynamic-scale quantization
//   mlir-tensorrt/compiler/lib/Backends/Kernel/KernelBackend.cpp:52-83
//   mlir-tensorrt/compiler/lib/Backends/Kernel/KernelSegmentation.cpp:53-113
// and scale = amax / maxbound as in tripy/examples/nanogpt/weight_loader.py:67-68.
// The reference's generated reduction has every thread walk a whole row serially
// (mlir-tensorrt/kernel/lib/Utils/TilingUtils.cpp:669-677); here the tensor is
// streamed once with 128-bit loads by a grid sized to the chip, reduced per wave
// with cross-lane exchanges, per workgroup through LDS, and across workgroups with
// a two-level tree of device-scope atomic max operations.  max is exact under any order, so the
// result is bit-identical to the sequential host reduction.
//
// abs/max run on the BIT PATTERN: for non-NaN floats, |x| orders like the unsigned
// integer (bits & 0x7fffffff), so v_and + v_max_u32 replace fabs + fmax and the
// bf16/f16 inputs need no conversion in the loop.  A NaN input yields a NaN amax
// (its pattern is the largest), unlike the host's std::max which would drop it
// (CoreModule.cpp:540-551); the programs this serves are NaN-free.
//
// scratch: (1 + 32) lines of 128 bytes owned by the caller's stream, each holding an
// (arrival ticket, running max) pair in its first eight bytes, all zero on entry; whoever arrives last at a
// pair restores its zeros, so back-to-back launches on one stream need no memset.
#include "common.hpp"

using namespace mtrt_dev;

namespace amax_cluster {

constexpr int kAmaxThreads = 256;
constexpr int kAmaxUnroll = 4;     // 128-bit loads in flight per lane per step
constexpr uint32_t kAmaxFanIn = 32;     // first-level groups of the cross-workgroup arrival tree
constexpr uint32_t kAmaxLineWords = 32; // one 128-byte line per (ticket, max) pair

template <typename X> struct AbsBits;
template <> struct AbsBits<F32> {  // returns max over the 4 floats, as f32 bit pattern
  static __device__ __forceinline__ uint32_t of(u32x4 t) {
    uint32_t a = t.x & 0x7FFFFFFFu, b = t.y & 0x7FFFFFFFu, c = t.z & 0x7FFFFFFFu, d = t.w & 0x7FFFFFFFu;
    a = a > b ? a : b; c = c > d ? c : d;
    return a > c ? a : c;
  }
  static __device__ __forceinline__ uint32_t one(const float* p) { return f32_to_bits(*p) & 0x7FFFFFFFu; }
  static __device__ __forceinline__ float finish(uint32_t m) { return bits_to_f32(m); }
  static constexpr int kPerVec = 4;
};
template <> struct AbsBits<BF16> { // 8 bf16 per vector; result kept as f32 bit pattern (bf16 << 16)
  static __device__ __forceinline__ uint32_t of(u32x4 t) {
    uint32_t m = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t lo = (t[j] << 16) & 0x7FFF0000u, hi = t[j] & 0x7FFF0000u;
      m = m > lo ? m : lo; m = m > hi ? m : hi;
    }
    return m;
  }
  static __device__ __forceinline__ uint32_t one(const uint16_t* p) { return (uint32_t(*p) << 16) & 0x7FFF0000u; }
  static __device__ __forceinline__ float finish(uint32_t m) { return bits_to_f32(m); }
  static constexpr int kPerVec = 8;
};
template <> struct AbsBits<F16> {  // 8 f16 per vector; result kept as f16 bit pattern
  static __device__ __forceinline__ uint32_t of(u32x4 t) {
    uint32_t m = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t lo = t[j] & 0x7FFFu, hi = (t[j] >> 16) & 0x7FFFu;
      m = m > lo ? m : lo; m = m > hi ? m : hi;
    }
    return m;
  }
  static __device__ __forceinline__ uint32_t one(const uint16_t* p) { return uint32_t(*p) & 0x7FFFu; }
  static __device__ __forceinline__ float finish(uint32_t m) { return f16_bits_to_f32(m); }
  static constexpr int kPerVec = 8;
};

// One arrival at a (ticket, max) pair: one 64-bit word, ticket count in the low half, running max in
// the high half.  Device-scope atomics execute at the memory side, the one place all eight XCDs agree
// on, so no cache write-back or invalidate is needed (an acquire/release pair at device scope would
// flush and invalidate the XCD's L2 once per workgroup).  Ordering is by completion: the 32-bit max on
// the high half RETURNS its old value and the empty asm consumes it, so the wave waits for that value
// before it issues the 64-bit add that takes the ticket; every max is therefore performed before the
// ticket of the same arrival, and all of them before the last ticket, whose add returns the whole old
// word: the last of `expected` arrivals finds the combined max in its high half (two dependent trips
// to memory per arrival instead of three).  Returns true for that arrival, with the max in `m`; it has
// also put the word back to zero.
__device__ __forceinline__ bool arrive(uint32_t* pair, uint32_t expected, uint32_t& m) {
  const uint32_t before = __hip_atomic_fetch_max(&pair[1], m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __asm__ volatile("" ::"v"(before) : "memory");
  unsigned long long* word = reinterpret_cast<unsigned long long*>(pair);
  const unsigned long long old = __hip_atomic_fetch_add(word, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (uint32_t(old) != expected - 1) return false;
  m = uint32_t(old >> 32);
  __hip_atomic_exchange(word, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return true;
}

template <typename X>
__device__ __forceinline__ void amax_body(const typename X::storage* __restrict__ x, int64_t n, float qmax,
                                          float* __restrict__ amax_out, float* __restrict__ scale_out,
                                          uint32_t* __restrict__ scratch) {
  using A = AbsBits<X>;
  // Elements before the first 16-byte boundary ("head") and after the last full
  // vector ("tail") are taken one per lane by workgroup 0; everything between is
  // streamed as 128-bit vectors, each workgroup owning one contiguous chunk.
  constexpr int kElemBytes = 16 / A::kPerVec;
  constexpr int64_t kStep = int64_t(kAmaxThreads) * kAmaxUnroll;
  int64_t head = int64_t((16u - uint32_t(reinterpret_cast<uintptr_t>(x) & 15u)) & 15u) / kElemBytes;
  head = head < n ? head : n;
  const int64_t nvec = (n - head) / A::kPerVec;
  const u32x4* __restrict__ xv = reinterpret_cast<const u32x4*>(x + head);
  // vectors per workgroup, rounded up; tensors below 2^32 vectors (64 GiB) take the 32-bit division (the 64-bit one is
  // a hundred scalar instructions in front of the first load)
  const uint64_t spread = uint64_t(nvec) + gridDim.x - 1;
  const int64_t share = (spread >> 32) == 0 ? int64_t(uint32_t(spread) / gridDim.x) : int64_t(spread / gridDim.x);
  const int64_t per = (share + kStep - 1) / kStep * kStep;                                  // chunk, whole steps
  const int64_t c0 = int64_t(blockIdx.x) * per;
  const int64_t c1 = c0 + per < nvec ? c0 + per : nvec;
  uint32_t m = 0;
  int64_t i = c0 + threadIdx.x;
  // kAmaxUnroll independent 128-bit loads per lane per trip
  for (; i + (kAmaxUnroll - 1) * kAmaxThreads < c1; i += kStep) {
    u32x4 t[kAmaxUnroll];
#pragma unroll
    for (int u = 0; u < kAmaxUnroll; ++u) t[u] = __builtin_nontemporal_load(xv + i + u * kAmaxThreads);
#pragma unroll
    for (int u = 0; u < kAmaxUnroll; ++u) { const uint32_t a = A::of(t[u]); m = m > a ? m : a; }
  }
  for (; i < c1; i += kAmaxThreads) { const uint32_t a = A::of(__builtin_nontemporal_load(xv + i)); m = m > a ? m : a; }
  if (blockIdx.x == 0 && threadIdx.x < 2 * A::kPerVec) {
    const int64_t tail0 = head + nvec * A::kPerVec;
    const int64_t e = threadIdx.x < A::kPerVec ? int64_t(threadIdx.x) : tail0 + (threadIdx.x - A::kPerVec);
    const bool live = threadIdx.x < A::kPerVec ? (e < head) : (e < n);
    if (live) { const uint32_t a = A::one(x + e); m = m > a ? m : a; }
  }

  m = wave_reduce(m, MaxU32());
  __shared__ uint32_t wave_max[kAmaxThreads / kWave];
  const int wave = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) wave_max[wave] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int w = 1; w < kAmaxThreads / kWave; ++w) m = m > wave_max[w] ? m : wave_max[w];
    // Two-level arrival tree: atomics on one address are served one after the other
    // by the memory side, so workgroups first meet in kAmaxFanIn groups (one cache
    // line each) and only the last of each group goes on to the root.
    const uint32_t groups = gridDim.x < kAmaxFanIn ? gridDim.x : kAmaxFanIn;
    const uint32_t g = blockIdx.x % groups;
    const uint32_t members = (gridDim.x - g + groups - 1) / groups;
    if (arrive(scratch + kAmaxLineWords * (1 + g), members, m) && arrive(scratch, groups, m)) {
      const float amax = A::finish(m);
      if (amax_out) *amax_out = amax;
      if (scale_out) *scale_out = amax / qmax;         // one IEEE divide, as the host does it
    }
  }
}

}  // namespace amax_cluster
using namespace amax_cluster;

// (x, n, qmax, amax_out, scale_out, scratch) ; x needs only its natural element alignment.
extern "C" __global__ void __launch_bounds__(kAmaxThreads) mtrt_amax_f32(
    const float* x, int64_t n, float qmax, float* amax_out, float* scale_out, uint32_t* scratch) {
  amax_body<F32>(x, n, qmax, amax_out, scale_out, scratch);
}
extern "C" __global__ void __launch_bounds__(kAmaxThreads) mtrt_amax_bf16(
    const uint16_t* x, int64_t n, float qmax, float* amax_out, float* scale_out, uint32_t* scratch) {
  amax_body<BF16>(x, n, qmax, amax_out, scale_out, scratch);
}
extern "C" __global__ void __launch_bounds__(kAmaxThreads) mtrt_amax_f16(
    const uint16_t* x, int64_t n, float qmax, float* amax_out, float* scale_out, uint32_t* scratch) {
  amax_body<F16>(x, n, qmax, amax_out, scale_out, scratch);
}
