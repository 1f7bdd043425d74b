// W8A8 GEMM cluster for gfx950:
//     acc[m,n] = sum_k i32(a[m,k]) * i32(w[k,n])                 (exact int32)
//     y[m,n]   = f16((f32(acc[m,n]) * a_scale[m]) * w_scale[n])   (two f32 roundings, then f16)
// i.e. the dot_general + per-token / per-output-channel dequantize epilogue of a
// quantized Linear (tripy/nvtripy/frontend/module/linear.py:112-151), which the
// reference realises as a plain FMA loop nest without matrix cores
// (mlir-tensorrt/kernel/test/Kernel/TransformSchedules/fallback-schedule-matmul.mlir:24).
//
// Matrix cores want both operands contiguous along K per row/column.  Activations
// [M,K] already are.  Weights arrive as [K,N] (N contiguous); they are constants of
// the program, so they are re-laid once into [N,K] by mtrt_w8_prepack_kn_to_nk and
// the GEMM consumes that.  The main loop (tiling, pipeline, LDS layout, tile order,
// epilogue staging) is the shared one in gemm_core.hpp with v_mfma_i32_32x32x32_i8.
#include "gemm_core.hpp"

namespace gemm_w8a8_cluster {

using namespace mtrt_dev;
using gemm_core::v4i;
typedef int v16i __attribute__((ext_vector_type(16)));

struct I8Traits {
  using Acc = v16i;
  using Scalar = int;
  static __device__ __forceinline__ Acc zero() {
    Acc z;
#pragma unroll
    for (int r = 0; r < 16; ++r) z[r] = 0;
    return z;
  }
  static __device__ __forceinline__ Acc mfma(v4i a, v4i b, Acc c) { return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0); }
};

// BN: columns of the workgroup's tile (the scratch holds 256 + BN floats)
template <int BN>
struct ScaleEpilogueT {
  const float* a_scale;
  const float* w_scale;
  const float* sa;                                   // a_scale of this tile's 256 rows, in LDS
  const float* sw;                                   // w_scale of this tile's BN columns, in LDS
  float as;
  __device__ __forceinline__ void setup(int8_t* scratch, int64_t m0, int64_t M, int64_t n0, int64_t N) {
    float* dst = reinterpret_cast<float*>(scratch);
    const int64_t row = m0 + threadIdx.x;              // the first 256 threads: 256 rows
    if (threadIdx.x < 256) dst[threadIdx.x] = row < M ? a_scale[row] : 0.0f;
    for (int c = threadIdx.x; c < BN; c += blockDim.x) dst[256 + c] = n0 + c < N ? w_scale[n0 + c] : 0.0f;
    sa = dst;
    sw = dst + 256;
  }
  __device__ __forceinline__ void row(int row_in_tile) { as = sa[row_in_tile]; }
  // the lane's column scales of one staging pass (HC column tiles of 32, four runs of four columns each), read from LDS
  // once and kept in registers for the pass's rows
  template <int HC>
  __device__ __forceinline__ void columns(int first_col_in_tile) {
#pragma unroll
    for (int jj = 0; jj < HC; ++jj)
#pragma unroll
      for (int q = 0; q < 4; ++q) wsr[jj][q] = *reinterpret_cast<const f32x4*>(sw + first_col_in_tile + jj * 32 + q * 8);
  }
  __device__ __forceinline__ void convert4(const v16i& acc, int q, int jj, uint32_t (&words)[2]) const {
#pragma unroll
    for (int e = 0; e < 4; e += 2)
      words[e >> 1] = f32x2_to_f16x2_bits((float(acc[4 * q + e]) * as) * wsr[jj][q][e], (float(acc[4 * q + e + 1]) * as) * wsr[jj][q][e + 1]);
  }
  f32x4 wsr[2][4];
};
using ScaleEpilogue = ScaleEpilogueT<256>;

// The entry points below have C linkage; they sit inside the namespace only so that
// its helper names do not meet those of the other clusters in the one-module build.

// (a [M,K] i8, w_nk [N,K] i8, a_scale [M] f32, w_scale [N] f32, y [M,N] f16, M, K, N, full_panels) ; K % 128 == 0,
// a and w_nk 16-byte aligned, both below 4 GiB.  The first full_panels * 256 columns are computed in
// 256 x 256 tiles, the rest in 256 x 128 tiles: with one workgroup per compute unit a launch runs in
// rounds, and a last round that would use few of the units is cut into twice as many tiles of half
// the length.  grid = even_blocks(full_panels * tiles_m) + even_blocks(half panels * tiles_m), block = 256 (each kind
// of tile dealt evenly to the XCDs, gemm_core::tile_of_even).
extern "C" __global__ void __launch_bounds__(gemm_core::THREADS, 1) mtrt_gemm_w8a8_nk(
    const int8_t* __restrict__ a, const int8_t* __restrict__ w, const float* __restrict__ a_scale,
    const float* __restrict__ w_scale, uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N, int64_t full_panels) {
  __shared__ __attribute__((aligned(16))) int8_t lds[gemm_core::LDS_BYTES];
  const int64_t tiles_m = (M + gemm_core::BM - 1) / gemm_core::BM;
  const int64_t full_blocks = gemm_core::even_blocks(full_panels * tiles_m);
  ScaleEpilogue epi{a_scale, w_scale, nullptr, nullptr, 0.0f, {}};
  int64_t tile_m, panel;
  if (int64_t(blockIdx.x) < full_blocks) {
    if (!gemm_core::tile_of_even(blockIdx.x, uint32_t(full_blocks), tiles_m, full_panels, tiles_m, tile_m, panel)) return;
    gemm_core::run<I8Traits, 4>(a, w, K, epi, y, M, N, K / gemm_core::BKB, tile_m * 256, panel * 256, lds);
  } else {
    const int64_t n_full = full_panels * 256;
    if (!gemm_core::tile_of_even(blockIdx.x - uint32_t(full_blocks), gridDim.x - uint32_t(full_blocks), tiles_m, (N - n_full + 127) / 128,
                                 tiles_m, tile_m, panel))
      return;
    gemm_core::run<I8Traits, 2>(a, w, K, epi, y, M, N, K / gemm_core::BKB, tile_m * 256, n_full + panel * 128, lds);
  }
}

// ---- weights straight into registers ---------------------------------------------------
// The loop above moves both operands through LDS with two 64 KiB stages, so the loads of a slice
// are issued only three k-steps before they are needed.  This kernel takes the WEIGHTS from a
// fragment-order re-layout straight into registers (two register sets, each k-step's registers
// re-filled seven k-steps before their next use) and leaves LDS to the activations alone: a ring
// of four 32 KiB stages filled by direct-to-LDS loads two slices ahead.  Four waves (2 x 2, one per
// SIMD), each 128 rows x 128 columns (JT = 4) or x 64 columns (JT = 2, the half-width tile of a last
// partial round): an activation fragment read from LDS serves four MFMAs.  The loop is written for
// 2 x NWN waves; with eight (2 x 4, two per SIMD, 128 x 64 each, twice the fragment reads) the launch is
// 3 % slower on the benchmark's data and 4 % on zero operands, measured in one process.
//
// What bounds it (measured on the eight-wave form, one MI355X at M=2048 K=4096 N=11008, counters per launch):
//   * with every load and LDS read taken out of the loop the launch still needs 164 k cycles per
//     XCD (ideal for its MFMAs: 98 k), with them 220 k; removing only the LDS reads or only the
//     barrier changes nothing, removing either operand's loads saves ~13 k, both ~56 k;
//   * making all workgroups load the same tile (everything L2-resident) changes nothing, making
//     all lanes of a load hit ONE cache line saves 36 k: the cost is per cache line requested by
//     the L1, not per byte, instruction or miss further out; the L1 reports "pending request"
//     stalls for 30 % of the launch (TCP_PENDING_STALL_CYCLES) at 24 B/clk/CU, less than half of
//     what the same L1 streams (60 B/clk/CU) when nothing else runs;
//   * the two waves that share a column half load the same weight lines; cacheable (not
//     nontemporal) weight loads let the second one hit and are 3 % faster.
// The tile already is as large as the register file allows, so the lines per MFMA cannot drop.
//
// Fragment order (mtrt_w8_prepack_frag): for each tile of 32 columns and each slice of 128 k, four
// 1 KiB blocks, one per k-step p; in a block lane l = 32*h + (n % 32) owns the 16 bytes
// k = 128*slice + 32*p + 16*h + [0..15] of column n: exactly the B operand of
// v_mfma_i32_32x32x32_i8 for that k-step, and every load instruction of a wave reads 1 KiB of
// contiguous memory.  Columns past N hold zeros.
namespace frag {

constexpr int kMW = 2;                                 // two rows of waves, 128 rows each
constexpr int kStageBytes = 256 * 128;                 // one slice of the activation panel
template <int NWN>
struct Waves {                                         // kMW x NWN waves
  static constexpr int kWaves = kMW * NWN, kThreads = 64 * kWaves;
  static constexpr int kG = 32 / kWaves;               // direct-to-LDS loads per wave and slice
  static constexpr int kOut = kWaves * gemm_core::kOutWave + 2048;
  static constexpr int kLds = kOut > 4 * kStageBytes ? kOut : 4 * kStageBytes;   // output staging, or the ring of four stages
};

template <int NWN, int JT, class Epilogue>
__device__ __forceinline__ void run(const int8_t* __restrict__ a, int64_t a_row_bytes, const v4i* __restrict__ wfrag,
                                    int64_t ntiles, Epilogue& epi, uint16_t* __restrict__ y, int64_t M, int64_t N,
                                    int64_t slices, int64_t m0, int64_t n0, int8_t* lds) {
  using namespace gemm_core;
  constexpr int kNWN = NWN, kWaves = Waves<NWN>::kWaves, kG = Waves<NWN>::kG;
  constexpr int kDmaPerStep = kG / 4;                  // direct-to-LDS loads per wave and k-step
  static_assert(kG % 4 == 0 && JT <= 4, "loads are dealt to the four chunks of a k-step");
  const int lane = threadIdx.x & 63;
  const int slot = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = slot / kNWN, wn = slot % kNWN;
  const int frow = lane & 31, fhalf = lane >> 5;

  v16i acc[4][JT];

  const uint32_t nslices = uint32_t(slices), last = nslices - 1;
  DmaLoaderT<kG> al;
  al.init(a, M, a_row_bytes, m0);
  v4i fa0[4], fa1[4];
  v4i raw[2][JT][4];
  // Every load takes a scalar base and a 32-bit lane offset (kept opaque, so that its widening is not hoisted out
  // of the loop: the load would then need a vector address pair and a 64-bit vector add of its own).
  const int8_t* wsrc[JT];                              // slice 0, k-step 0 of each column tile (uniform)
  uint32_t wlane = uint32_t(lane) * 16;
#pragma unroll
  for (int j = 0; j < JT; ++j) {
    int64_t tile = n0 / 32 + wn * JT + j;
    tile = tile < ntiles ? tile : ntiles - 1;          // tiles past N: some valid data, never stored
    wsrc[j] = reinterpret_cast<const int8_t*>(wfrag + tile * slices * 256);
  }
  auto fetch_one = [&](auto set, int j, uint32_t slice, int p) {
    constexpr int SET = decltype(set)::value;
    __asm__ volatile("" : "+v"(wlane));
    raw[SET][j][p] = *reinterpret_cast<const v4i*>(wsrc[j] + (uint64_t(slice) * 4096 + uint32_t(p) * 1024) + wlane);
  };
  // Fragment reads are opaque instructions, waited for by count: the reads form one stream (chunk c of a k-step
  // reads row tile c of the next k-step), so when chunk c needs its fragment exactly three younger reads are
  // outstanding.  Left to the compiler, every k-step got an s_waitcnt lgkmcnt(0) right behind a read that had
  // just been issued (one exposed LDS round trip per k-step).  Row tile i sits i * 4096 bytes further; the
  // swizzle depends on the lane and the k chunk only.
  const uint32_t lds_base = uint32_t(uintptr_t((lds_void_t*)lds));
  uint32_t a_lane[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) a_lane[p] = lds_base + uint32_t(lds_off(wm * 128 + frow, 2 * p + fhalf));
  auto read_a = [&](v4i (&f)[4], uint32_t addr, auto tile) {
    constexpr int I = decltype(tile)::value;
    __asm__ volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(f[I]) : "v"(addr), "n"(I * 4096) : "memory");
  };
  auto landed_a = [&](v4i (&f)[4], int i) { __asm__ volatile("s_waitcnt lgkmcnt(3)" : "+v"(f[i])::"memory"); };
  auto stage_off = [&](uint32_t slice) { return uint32_t(slice & 3) * uint32_t(kStageBytes); };
  auto stage = [&](uint32_t slice) { return lds + stage_off(slice); };
  auto at_most_last = [&](uint32_t slice) { return slice - ((uint32_t(last - slice) >> 31) * (slice - last)); };  // scalar min

  const uint32_t one = at_most_last(1);
  // what slice 0 needs first, then slice 1
#pragma unroll
  for (int g = 0; g < kG; ++g) al.dma_at(al.slice_base(0), stage(0), g);
#pragma unroll
  for (int p = 0; p < 4; ++p)
#pragma unroll
    for (int j = 0; j < JT; ++j) fetch_one(IntC<0>{}, j, 0, p);
#pragma unroll
  for (int g = 0; g < kG; ++g) al.dma_at(al.slice_base(one), stage(1), g);
#pragma unroll
  for (int p = 0; p < 3; ++p)                          // k-step 3 of slice 1 is fetched in k-step 0 of slice 0
#pragma unroll
    for (int j = 0; j < JT; ++j) fetch_one(IntC<1>{}, j, one, p);
  __builtin_amdgcn_sched_barrier(0);                   // (all of them issued here, none moved behind the barrier)
  // The accumulators are cleared by the matrix cores themselves (0 x 0 + 0) while those loads are under way; written as
  // plain zeros the clearing (one register move per accumulator register) ends up behind the barrier, in front of the loop.
  {
    v4i none = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < JT; ++j) {
        __asm__ volatile("" : "+v"(none));             // one MFMA per accumulator, not one result copied around
        acc[i][j] = I8Traits::mfma(none, none, I8Traits::zero());
      }
    __builtin_amdgcn_sched_barrier(0);
  }
  drain_and_barrier();                                 // (starting on slice 0 while slice 1 is still under way: 3 % slower)
  read_a(fa0, a_lane[0] + stage_off(0), IntC<0>{});
  read_a(fa0, a_lane[0] + stage_off(0), IntC<1>{});
  read_a(fa0, a_lane[0] + stage_off(0), IntC<2>{});
  read_a(fa0, a_lane[0] + stage_off(0), IntC<3>{});

  // k-step T of slice s (parity PAR): four fenced chunks; chunk c multiplies row tile c by the JT
  // weight fragments of this k-step and carries one A fragment read for the next k-step.  The
  // memory instructions are spread EVENLY over the k-steps (issued in bursts they queue up in
  // front of the L1, whose 64 B/clk this loop uses to three quarters, and the waves behind them
  // stall): each k-step issues one direct-to-LDS load of slice s+2 and JT weight loads into the
  // registers the PREVIOUS k-step finished with: k-step T >= 1 re-fills k-step T-1's registers
  // of this parity for slice s+2, k-step 0 re-fills k-step 3's registers of the other parity for
  // slice s+1.
  auto kstep = [&](auto par, auto step, v4i (&cur)[4], v4i (&nxt)[4], uint32_t ra, uint32_t s1, uint32_t s2, const int8_t* src,
                   int8_t* nd) {
    constexpr int PAR = decltype(par)::value, T = decltype(step)::value;
    const uint32_t raddr = a_lane[(T + 1) & 3] + ra;
    auto chunk = [&](auto cc) {
      constexpr int c = decltype(cc)::value;
      landed_a(cur, c);
#pragma unroll
      for (int j = 0; j < JT; ++j) acc[c][j] = I8Traits::mfma(raw[PAR][j][T], cur[c], acc[c][j]);
      read_a(nxt, raddr, cc);
      if (c % 2 == 0 && c / 2 < kDmaPerStep) al.dma_at(src, nd, T * kDmaPerStep + c / 2);
      constexpr int j = JT == 4 ? c : c - 1;             // column tile whose weights this chunk fetches
      if (j >= 0 && j < JT) {
        if (T == 0) fetch_one(IntC<PAR ^ 1>{}, j, s1, 3);
        else fetch_one(par, j, s2, T - 1);
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    chunk(IntC<0>{});
    chunk(IntC<1>{});
    chunk(IntC<2>{});
    chunk(IntC<3>{});
  };
  auto slice_body = [&](auto par, uint32_t s) {
    const uint32_t pa = stage_off(s);
    const uint32_t s1 = at_most_last(s + 1), s2 = at_most_last(s + 2);
    const int8_t* src = al.slice_base(s2);
    int8_t* nd = stage(s + 2);
    kstep(par, IntC<0>{}, fa0, fa1, pa, s1, s2, src, nd);
    kstep(par, IntC<1>{}, fa1, fa0, pa, s1, s2, src, nd);
    kstep(par, IntC<2>{}, fa0, fa1, pa, s1, s2, src, nd);
    // everything issued before this slice has landed (the panel of slice s+1 and its weights for
    // k-steps 0..2); the loads of this slice's first three k-steps may still fly
    // (the fragment reads in flight belong to a stage that is not written before the next barrier but one)
    constexpr int kFly = 3 * kDmaPerStep + 3 * JT;
    __builtin_amdgcn_s_waitcnt(0x0F70 | (kFly & 15) | ((kFly >> 4) << 14));   // vmcnt(kFly)
    __asm__ volatile("s_barrier" ::: "memory");
    kstep(par, IntC<3>{}, fa1, fa0, stage_off(s + 1), s1, s2, src, nd);
  };

  uint32_t s = 0;
  for (; s + 1 < nslices; s += 2) {
    slice_body(IntC<0>{}, s);
    slice_body(IntC<1>{}, s + 1);
  }
  if (s < nslices) slice_body(IntC<0>{}, s);
  __builtin_amdgcn_s_waitcnt(0x0070);                  // the surplus loads of the last slices have landed
  // ... and so have the surplus fragment reads: their registers stay allocated up to here
#pragma unroll
  for (int i = 0; i < 4; ++i) __asm__ volatile("s_waitcnt lgkmcnt(0)" ::"v"(fa0[i]), "v"(fa1[i]) : "memory");

  write_tile<JT, kNWN, kWaves>(acc, epi, y, M, N, m0, n0, lds, slot, true);
}


// ---- 256 x 384 tiles: four waves of 256 x 96 -------------------------------------------------------------
// The widest tile the register file holds: 384 accumulator registers per lane.  Every wave owns all 256 rows of 96
// columns, so each weight fragment is loaded by ONE wave (the 2 x 2 waves above load each twice) and a workgroup
// moves 80 KiB per slice for 384 MFMAs where the 256 x 256 tile moves 96 KiB for 256: on zero operands the loop runs at
// 95 % of its MFMA time.  What it takes:
//   * With one wave per SIMD the compiler gives the matrix instructions accumulation registers only, 256 per lane.
//     The third column tile's accumulators therefore live in ordinary vector registers, through MFMAs written as
//     instructions (the compiler does not see inside: s_nops in front of the epilogue let the matrix cores finish).
//   * That leaves about 120 vector registers for everything else.  Activation fragments are read HALF a k-step
//     ahead (two sets of four: chunks 0..3 of a k-step read its row tiles 4..7, chunks 4..7 row tiles 0..3 of the
//     next k-step); the weights of a k-step (3 x 16 bytes per lane) sit in a ring of four k-steps and are asked for
//     again as soon as the k-step is over, three k-steps before their next use.
//   * Memory instructions are issued in a fixed order per k-step (chunk 0: activations, chunks 1..3: weights,
//     chunk 4: activations) and waited for by count: when a k-step starts, eleven have been issued since its weights
//     were asked for; the activations of slice s+1 were asked for during slice s-1 and have landed by the same count
//     in front of k-step 3, where the workgroup meets.
// Measured against mtrt_gemm_w8a8_frag in one process at M = 2048, K = 4096, N = 11008 (232 tiles, one round, against
// 1.5 rounds of the smaller tile): 83.5 -> 77.9 us on the benchmark's data, 64.0 -> 58.1 us on zeros, same bits.
constexpr int kWideBN = 384;
constexpr int kWideOut = 4 * gemm_core::kOutWave + (256 + kWideBN) * 4;
constexpr int kWideLds = kWideOut > 4 * kStageBytes ? kWideOut : 4 * kStageBytes;

template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(gemm_core::IntC<I>{});
    static_for<I + 1, N>(f);
  }
}
// 16 bytes per lane of k-step T of a weight slice: scalar base, 32-bit lane offset, the k-step as the instruction's offset
template <int T>
__device__ __forceinline__ void load_w(v4i& dst, uint32_t lane_off, const int8_t* base) {
  __asm__ volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(dst) : "v"(lane_off), "s"(base), "n"(T * 1024) : "memory");
}

template <class Epilogue>
__device__ __forceinline__ void run_wide(const int8_t* __restrict__ a, int64_t a_row_bytes, const v4i* __restrict__ wfrag,
                                         int64_t ntiles, Epilogue& epi, uint16_t* __restrict__ y, int64_t M, int64_t N,
                                         int64_t slices, int64_t m0, int64_t n0, int8_t* lds) {
  using namespace gemm_core;
  constexpr int IT = 8, JT = 3, AN = 4, kG = 8;
  constexpr int JA = 2;                                // column tiles whose accumulators the compiler places
  constexpr int kFly = 11;                             // memory instructions issued since a k-step's weights were asked for
  const int lane = threadIdx.x & 63;
  const int slot = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // = the wave's column: 1 x 4 waves
  const int frow = lane & 31, fhalf = lane >> 5;

  v16i acc[IT][JT];
  const uint32_t nslices = uint32_t(slices), last = nslices - 1;
  DmaLoaderT<kG> al;
  al.init(a, M, a_row_bytes, m0);
  v4i fa[2][AN];
  v4i wr[4][JT];
  const int8_t* wsrc[JT];                              // slice 0 of each column tile (uniform)
  uint32_t wlane = uint32_t(lane) * 16;
#pragma unroll
  for (int j = 0; j < JT; ++j) {
    int64_t tile = n0 / 32 + slot * JT + j;
    tile = tile < ntiles ? tile : ntiles - 1;          // tiles past N: some valid data, never stored
    wsrc[j] = reinterpret_cast<const int8_t*>(wfrag + tile * slices * 256);
  }
  auto fetch_w = [&](auto tt, v4i& dst, int j, uint32_t slice) {
    load_w<decltype(tt)::value>(dst, wlane, wsrc[j] + uint64_t(slice) * 4096);
  };
  const uint32_t lds_base = uint32_t(uintptr_t((lds_void_t*)lds));
  uint32_t a_lane[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) a_lane[p] = lds_base + uint32_t(lds_off(frow, 2 * p + fhalf));
  auto read_a = [&](v4i& dst, uint32_t addr, auto tile) {
    constexpr int I = decltype(tile)::value;
    __asm__ volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(I * 4096) : "memory");
  };
  // the reads form one stream, four chunks ahead of their use: three younger ones may be outstanding
  auto landed_a = [&](v4i& frag) { __asm__ volatile("s_waitcnt lgkmcnt(3)" : "+v"(frag)::"memory"); };
  auto stage_off = [&](uint32_t slice) { return uint32_t(slice & 3) * uint32_t(kStageBytes); };
  auto stage = [&](uint32_t slice) { return lds + stage_off(slice); };
  auto at_most_last = [&](uint32_t slice) { return slice - ((uint32_t(last - slice) >> 31) * (slice - last)); };  // scalar min

  // slice 0 and its weights for k-steps 0..2 (k-step 3's are asked for in k-step 0, like every slice's), then slice 1
  const uint32_t one = at_most_last(1);
#pragma unroll
  for (int g = 0; g < kG; ++g) al.dma_at(al.slice_base(0), stage(0), g);
  static_for<0, 3>([&](auto t) {
    constexpr int T = decltype(t)::value;
#pragma unroll
    for (int j = 0; j < JT; ++j) fetch_w(t, wr[T][j], j, 0);
  });
#pragma unroll
  for (int g = 0; g < kG; ++g) al.dma_at(al.slice_base(one), stage(1), g);
  __builtin_amdgcn_sched_barrier(0);
  {                                                    // accumulators cleared by the matrix cores under those loads
    v4i none = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < IT; ++i)
#pragma unroll
      for (int j = 0; j < JT; ++j) {
        __asm__ volatile("" : "+v"(none));
        if (j < JA) acc[i][j] = I8Traits::mfma(none, none, I8Traits::zero());
        else __asm__ volatile("v_mfma_i32_32x32x32_i8 %0, %1, %1, 0" : "=v"(acc[i][j]) : "v"(none));
      }
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int t = 0; t < 3; ++t) __asm__ volatile("s_waitcnt vmcnt(0)" : "+v"(wr[t][0]), "+v"(wr[t][1]), "+v"(wr[t][2])::"memory");
  drain_and_barrier();
  static_for<0, AN>([&](auto i) { read_a(fa[0][decltype(i)::value], a_lane[0] + stage_off(0), i); });

  // k-step T of slice s0 (the next slice: s1): eight fenced chunks; chunk c multiplies row tile c by the three weight
  // fragments of the k-step.  ca: LDS offset of the stage this k-step reads, ra: of the stage the next k-step reads.
  auto kstep = [&](auto step, uint32_t ca, uint32_t ra, uint32_t s0, uint32_t s1, const int8_t* src, int8_t* nd) {
    constexpr int T = decltype(step)::value;
    const uint32_t raddr = a_lane[(T + 1) & 3] + ra, caddr = a_lane[T] + ca;
    __asm__ volatile("s_waitcnt vmcnt(%3)" : "+v"(wr[T][0]), "+v"(wr[T][1]), "+v"(wr[T][2]) : "n"(kFly) : "memory");
    static_for<0, IT>([&](auto cc) {
      constexpr int c = decltype(cc)::value;
      constexpr int ASET = c / AN, AI = c % AN;
      landed_a(fa[ASET][AI]);
#pragma unroll
      for (int j = 0; j < JT; ++j) {
        if (j < JA) acc[c][j] = I8Traits::mfma(wr[T][j], fa[ASET][AI], acc[c][j]);
        else __asm__ volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(acc[c][j]) : "v"(wr[T][j]), "v"(fa[ASET][AI]));
      }
      if constexpr (c < AN) read_a(fa[1][c], caddr, IntC<c + AN>{});           // row tile c + 4 of this k-step
      else read_a(fa[0][c - AN], raddr, IntC<c - AN>{});                       // row tile c - 4 of the next
      if constexpr (c == 0) al.dma_at(src, nd, 2 * T);
      if constexpr (c == 4) al.dma_at(src, nd, 2 * T + 1);
      if constexpr (c >= 1 && c <= 3) {                // the registers of the k-step before this one, for their next use
        if constexpr (T == 0) fetch_w(IntC<3>{}, wr[3][c - 1], c - 1, s0);
        else fetch_w(IntC<T - 1>{}, wr[T - 1][c - 1], c - 1, s1);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  for (uint32_t s = 0; s < nslices; ++s) {
    const uint32_t pa = stage_off(s);
    const uint32_t s1 = at_most_last(s + 1), s2 = at_most_last(s + 2);
    const int8_t* src = al.slice_base(s2);             // the slice fetched during this one (past the end: the last again,
    int8_t* nd = stage(s + 2);                         //  into a stage nobody reads)
    kstep(IntC<0>{}, pa, pa, s, s1, src, nd);
    kstep(IntC<1>{}, pa, pa, s, s1, src, nd);
    kstep(IntC<2>{}, pa, pa, s, s1, src, nd);
    // the activations of slice s+1 have landed (fifteen memory instructions were issued since the last of them); the
    // fragment reads in flight belong to stages that are not written before the next barrier but one
    __asm__ volatile("s_waitcnt vmcnt(%0)" ::"n"(kFly) : "memory");
    __asm__ volatile("s_barrier" ::: "memory");
    kstep(IntC<3>{}, pa, stage_off(s + 1), s, s1, src, nd);
  }
  __builtin_amdgcn_s_waitcnt(0x0070);                  // the surplus loads and fragment reads have landed: their
#pragma unroll                                         // registers stay allocated up to here
  for (int i = 0; i < AN; ++i) __asm__ volatile("s_waitcnt lgkmcnt(0)" ::"v"(fa[0][i]), "v"(fa[1][i]) : "memory");
#pragma unroll
  for (int t = 0; t < 4; ++t) __asm__ volatile("s_waitcnt vmcnt(0)" ::"v"(wr[t][0]), "v"(wr[t][1]), "v"(wr[t][2]) : "memory");
  __asm__ volatile("s_nop 15\n\ts_nop 15" ::: "memory");   // the matrix cores are done with the accumulators in vector registers

  write_tile<JT, 4, 4>(acc, epi, y, M, N, m0, n0, lds, slot, true);
}

}  // namespace frag

// (a [M,K] i8, w_frag (fragment order), a_scale [M] f32, w_scale [N] f32, y [M,N] f16, M, K, N, full_panels) ;
// K % 128 == 0, a and w_frag 16-byte aligned, a below 4 GiB.  Tiles and grid as mtrt_gemm_w8a8_nk
// (256 x 256 for the first full_panels * 256 columns, 256 x 128 after), block = 64 * 2 * NWN.
template <int NWN>
__device__ __forceinline__ void frag_kernel(const int8_t* __restrict__ a, const v4i* __restrict__ w_frag, const float* __restrict__ a_scale,
                                            const float* __restrict__ w_scale, uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N,
                                            int64_t full_panels, int8_t* lds) {
  constexpr int JT = 8 / NWN;                          // column tiles per wave in a full tile; half of it in a half tile
  const int64_t tiles_m = (M + 255) / 256, ntiles = (N + 31) / 32;
  const int64_t full_blocks = gemm_core::even_blocks(full_panels * tiles_m);
  ScaleEpilogue epi{a_scale, w_scale, nullptr, nullptr, 0.0f, {}};
  int64_t tile_m, panel;
  if (int64_t(blockIdx.x) < full_blocks) {
    if (!gemm_core::tile_of_even(blockIdx.x, uint32_t(full_blocks), tiles_m, full_panels, tiles_m, tile_m, panel)) return;
    frag::run<NWN, JT>(a, K, w_frag, ntiles, epi, y, M, N, K / 128, tile_m * 256, panel * 256, lds);
  } else {
    const int64_t n_full = full_panels * 256;
    if (!gemm_core::tile_of_even(blockIdx.x - uint32_t(full_blocks), gridDim.x - uint32_t(full_blocks), tiles_m, (N - n_full + 127) / 128,
                                 tiles_m, tile_m, panel))
      return;
    frag::run<NWN, JT / 2>(a, K, w_frag, ntiles, epi, y, M, N, K / 128, tile_m * 256, n_full + panel * 128, lds);
  }
}
// Four waves, 2 x 2, each 128 rows x 128 columns (one per SIMD): an activation fragment read from LDS serves four MFMAs.
extern "C" __global__ void __launch_bounds__(frag::Waves<2>::kThreads, 1) mtrt_gemm_w8a8_frag(
    const int8_t* __restrict__ a, const v4i* __restrict__ w_frag, const float* __restrict__ a_scale,
    const float* __restrict__ w_scale, uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N, int64_t full_panels) {
  __shared__ __attribute__((aligned(16))) int8_t lds[frag::Waves<2>::kLds];
  frag_kernel<2>(a, w_frag, a_scale, w_scale, y, M, K, N, full_panels, lds);
}
// 256 x 384 tiles (frag::run_wide).  (a, w_frag, a_scale, w_scale, y, M, K, N) as above.
// grid = 8 * ceil(ceil(M/256) * ceil(N/384) / 8), block = 256: the tiles dealt evenly to the XCDs, a panel's M tiles neighbours.
extern "C" __global__ void __launch_bounds__(256, 1) mtrt_gemm_w8a8_frag_t256x384(
    const int8_t* __restrict__ a, const v4i* __restrict__ w_frag, const float* __restrict__ a_scale,
    const float* __restrict__ w_scale, uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N) {
  __shared__ __attribute__((aligned(16))) int8_t lds[frag::kWideLds];
  const int64_t tiles_m = (M + 255) / 256, ntiles = (N + 31) / 32, panels = (N + frag::kWideBN - 1) / frag::kWideBN;
  ScaleEpilogueT<frag::kWideBN> epi{a_scale, w_scale, nullptr, nullptr, 0.0f, {}};
  int64_t tile_m, panel;
  if (!gemm_core::tile_of_even(blockIdx.x, gridDim.x, tiles_m, panels, tiles_m, tile_m, panel)) return;
  frag::run_wide(a, K, w_frag, ntiles, epi, y, M, N, K / 128, tile_m * 256, panel * frag::kWideBN, lds);
}
// Weight re-layout into fragment order, from [K,N] (nk = 0) or [N,K] (nk = 1).  One 16-byte chunk per
// thread.  (w, w_frag, K, N, nk) ; K % 128 == 0 ; w_frag holds 32 * ceil(N/32) * K bytes.
extern "C" __global__ void __launch_bounds__(256) mtrt_w8_prepack_frag(const int8_t* __restrict__ w, v4i* __restrict__ w_frag,
                                                                     int64_t K, int64_t N, int32_t nk) {
  const int64_t slices = K / 128, ntiles = (N + 31) / 32;
  const int64_t total = ntiles * slices * 256;
  for (int64_t id = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; id < total; id += int64_t(gridDim.x) * blockDim.x) {
    const int lane = int(id & 63), p = int((id >> 6) & 3);
    const int64_t slice = (id >> 8) % slices, tile = (id >> 8) / slices;
    const int64_t n = tile * 32 + (lane & 31), k0 = slice * 128 + 32 * p + 16 * (lane >> 5);
    union { v4i v; int8_t b[16]; } c;
#pragma unroll
    for (int i = 0; i < 16; ++i) c.b[i] = n < N ? (nk ? w[n * K + k0 + i] : w[(k0 + i) * N + n]) : int8_t(0);
    w_frag[id] = c.v;
  }
}

// ---- small M (<= 32): one workgroup per 32 columns, four waves split K -----------------------------------
// A launch of the tile kernel above lasts one tile's whole K loop however few rows it has (M = 16 at K = 4096,
// N = 11008: 21.7 us) although all it has to do is read the weights once (45 MB).  Here every workgroup owns one
// tile of 32 columns (or two, see small_m_tiles) over all of K, its four waves a quarter of K each: a wave keeps
// a ring of four stages (8 * G rows x 128 k of activations each) of its own in LDS, filled by direct-to-LDS loads
// three slices ahead as whole 128-byte row segments (a fragment read straight from memory would touch 32 cache
// lines), and takes the weights from fragment order straight into registers: no barrier until the four partial
// sums (int32, exact in any order) meet in LDS.  G: groups of 8 activation rows per stage (M <= 8 * G).
namespace small_m {

template <int G, int WAVES, int JT>
__device__ __forceinline__ void run(const int8_t* __restrict__ a, const v4i* __restrict__ wfrag, const float* __restrict__ a_scale,
                                    const float* __restrict__ w_scale, uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N,
                                    int8_t* lds) {
  constexpr int kStages = 4, kStageBytes = 8 * G * 128;
  constexpr int kLoads = G + 4 * JT;                 // memory instructions per slice and wave
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int frow = lane & 31, fhalf = lane >> 5;
  const int64_t slices = K / 128;
  const int64_t kb0 = slices * wave / WAVES, kb1 = slices * (wave + 1) / WAVES;
  int64_t tile[JT];
  const v4i* bp[JT];
#pragma unroll
  for (int j = 0; j < JT; ++j) {
    tile[j] = blockIdx.x + int64_t(j) * gridDim.x;
    bp[j] = wfrag + (tile[j] * slices) * 256 + lane;
  }
  int8_t* ring = lds + wave * (kStages * kStageBytes);

  // direct-to-LDS load g (of G) of a slice: rows 8g .. 8g+7, lane l <-> (row l >> 3, LDS chunk l & 7)
  uint32_t aoff[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const int lrow = g * 8 + (lane >> 3);
    const int64_t row = lrow < M ? lrow : M - 1;     // rows past M repeat the last row; never stored
    aoff[g] = uint32_t(row * K + (((lane & 7) ^ ((lrow >> 1) & 7)) << 4));
  }
  struct Slice {
    v4i w[JT][4];
  };
  // everything slice kb needs from memory: G + 4 JT loads, always, so that the waits can count
  auto fetch = [&](int64_t kb, int64_t clamp, Slice& dst) {
    kb = kb < clamp ? kb : clamp;
    int8_t* st = ring + int(kb & (kStages - 1)) * kStageBytes;
#pragma unroll
    for (int g = 0; g < G; ++g)
      __builtin_amdgcn_global_load_lds((gemm_core::global_void_t*)(a + kb * 128 + aoff[g]),
                                       (gemm_core::lds_void_t*)(st + g * 1024), 16, 0, 0);
    // register loads as opaque instructions, the waits placed by hand in `landed` (the compiler's own
    // bookkeeping drains every load carried around a loop before its first use)
#pragma unroll
    for (int j = 0; j < JT; ++j)
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const v4i* wsrc = bp[j] + kb * 256 + p * 64;
        __asm__ volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(dst.w[j][p]) : "v"(wsrc) : "memory");
      }
  };
  // four slices issued, the loads of three may fly -> those of the oldest slice have landed
  auto landed = [&](Slice& sl) {
#pragma unroll
    for (int j = 0; j < JT; ++j)
#pragma unroll
      for (int p = 0; p < 4; ++p) __asm__ volatile("s_waitcnt vmcnt(%1)" : "+v"(sl.w[j][p]) : "n"(3 * kLoads) : "memory");
  };
  auto landed_all = [&](Slice& sl) {
#pragma unroll
    for (int j = 0; j < JT; ++j)
#pragma unroll
      for (int p = 0; p < 4; ++p) __asm__ volatile("s_waitcnt vmcnt(0)" : "+v"(sl.w[j][p])::"memory");
  };

  v16i acc[JT];
#pragma unroll
  for (int j = 0; j < JT; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0;
  auto multiply = [&](int64_t kb, const Slice& sl) {
    const int8_t* st = ring + int(kb & (kStages - 1)) * kStageBytes;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int arow = frow < 8 * G ? frow : 8 * G - 1;   // rows past the ring: any valid data, never stored
      const v4i fa = *reinterpret_cast<const v4i*>(st + gemm_core::lds_off(arow, 2 * p + fhalf));
#pragma unroll
      for (int j = 0; j < JT; ++j) acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, sl.w[j][p], acc[j], 0, 0, 0);
    }
  };

  // Main part: groups of four slices with four register sets, so that nothing is copied (a copy would have
  // to wait for the load) and the loop has no branch; three slices stay in flight.
  const int64_t kmain = kb0 + ((kb1 - kb0) & ~int64_t(3));
  if (kb0 < kmain) {
    const int64_t clamp = kmain - 1;                   // past the end: the last slice again, into a stage nobody reads
    Slice s0, s1, s2, s3;
    fetch(kb0, clamp, s0);
    fetch(kb0 + 1, clamp, s1);
    fetch(kb0 + 2, clamp, s2);
    for (int64_t kb = kb0; kb < kmain; kb += 4) {
      fetch(kb + 3, clamp, s3);
      landed(s0);
      multiply(kb, s0);
      fetch(kb + 4, clamp, s0);
      landed(s1);
      multiply(kb + 1, s1);
      fetch(kb + 5, clamp, s1);
      landed(s2);
      multiply(kb + 2, s2);
      fetch(kb + 6, clamp, s2);
      landed(s3);
      multiply(kb + 3, s3);
    }
    // the surplus loads of the last group still target these registers: keep them until they land
    landed_all(s0);
    landed_all(s1);
    landed_all(s2);
  }
  for (int64_t kb = kmain; kb < kb1; ++kb) {           // at most three slices, one at a time
    Slice sl;
    __builtin_amdgcn_s_waitcnt(0x0070);
    fetch(kb, kb, sl);
    landed_all(sl);
    multiply(kb, sl);
  }
  __builtin_amdgcn_s_waitcnt(0x0070);                  // surplus loads have landed before the ring is reused
  int (*partial)[16][64] = reinterpret_cast<int (*)[16][64]>(lds);
#pragma unroll
  for (int j = 0; j < JT; ++j) {
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 16; ++r) partial[wave][r][lane] = acc[j][r];
    __syncthreads();
    for (int e = threadIdx.x; e < 16 * 64; e += 64 * WAVES) {
      const int r = e >> 6, l = e & 63;
      int v = partial[0][r][l];
#pragma unroll
      for (int w = 1; w < WAVES; ++w) v = v + partial[w][r][l];
      const int64_t row = (r >> 2) * 8 + (l >> 5) * 4 + (r & 3);
      const int64_t c = tile[j] * 32 + (l & 31);
      if (row < M && c < N) y[row * N + c] = uint16_t(f32_to_f16_bits((float(v) * a_scale[row]) * w_scale[c]));
    }
  }
}

// The grid is one workgroup per column tile, or, while that would leave some compute units with two workgroups
// and the rest with one (tiles between one and two times the compute units), one workgroup per compute unit:
// workgroup g then also takes tile g + gridDim.x if there is one, and reads the activations once for both.
template <int G>
__device__ __forceinline__ void tiles(const int8_t* __restrict__ a, const v4i* __restrict__ wfrag, const float* __restrict__ a_scale,
                                      const float* __restrict__ w_scale, uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N,
                                      int8_t* lds) {
  const int64_t ntiles = (N + 31) / 32;
  if (int64_t(blockIdx.x) + gridDim.x < ntiles)
    run<G, 4, 2>(a, wfrag, a_scale, w_scale, y, M, K, N, lds);
  else
    run<G, 4, 1>(a, wfrag, a_scale, w_scale, y, M, K, N, lds);
}

}  // namespace small_m

// (a [M,K] i8, w_frag (fragment order), a_scale [M] f32, w_scale [N] f32, y [M,N] f16, M, K, N) ; K % 128 == 0, a and
// w_frag 16-byte aligned, M * K < 2^32; grid = ceil(N / 32) or the number of compute units (see small_m::tiles), block = 256.
// M <= 16:
extern "C" __global__ void __launch_bounds__(256) mtrt_gemm_w8a8_small16(
    const int8_t* __restrict__ a, const v4i* __restrict__ w_frag, const float* __restrict__ a_scale,
    const float* __restrict__ w_scale, uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N) {
  __shared__ __attribute__((aligned(16))) int8_t lds[4 * 4 * 2 * 1024];
  small_m::tiles<2>(a, w_frag, a_scale, w_scale, y, M, K, N, lds);
}
// Any K (no alignment needs): one output element per lane, plain loops.  Only K = 0 is left to it (every
// other shape runs on the matrix cores).
extern "C" __global__ void __launch_bounds__(256) mtrt_gemm_w8a8_nk_any(
    const int8_t* __restrict__ a, const int8_t* __restrict__ w, const float* __restrict__ a_scale,
    const float* __restrict__ w_scale, uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N) {
  const int64_t total = M * N;
  for (int64_t e = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; e < total; e += int64_t(gridDim.x) * blockDim.x) {
    const int64_t m = e / N, n = e - m * N;
    int acc = 0;
    for (int64_t k = 0; k < K; ++k) acc += int(a[m * K + k]) * int(w[n * K + k]);
    y[e] = uint16_t(f32_to_f16_bits((float(acc) * a_scale[m]) * w_scale[n]));
  }
}

// Up to 32 rows on [N,K] weights read as whole rows (gemm_core::rows32): (a [M,K] i8, w_nk [N,K] i8, a_scale, w_scale, y,
// M <= 32, K, N) ; K % 128 == 0, a and w_nk 16-byte aligned; grid: any, block = 512.
struct RowsScaleEpilogue {
  const float* a_scale;
  const float* w_scale;
  __device__ __forceinline__ uint32_t finish(int sum, int64_t row, int64_t col) const {
    return f32_to_f16_bits((float(sum) * a_scale[row]) * w_scale[col]);
  }
};
extern "C" __global__ void __launch_bounds__(512) mtrt_gemm_w8a8_nk_rows32(
    const int8_t* __restrict__ a, const int8_t* __restrict__ w_nk, const float* __restrict__ a_scale,
    const float* __restrict__ w_scale, uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N) {
  __shared__ __attribute__((aligned(16))) int8_t lds[gemm_core::rows32::lds_bytes<8>()];
  RowsScaleEpilogue epi{a_scale, w_scale};
  gemm_core::rows32::run<I8Traits, 8>(a, w_nk, K, epi, y, M, N, lds);
}
// ... and up to 64 rows: two activation row tiles against each weight fragment
extern "C" __global__ void __launch_bounds__(512) mtrt_gemm_w8a8_nk_rows64(
    const int8_t* __restrict__ a, const int8_t* __restrict__ w_nk, const float* __restrict__ a_scale,
    const float* __restrict__ w_scale, uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N) {
  __shared__ __attribute__((aligned(16))) int8_t lds[gemm_core::rows32::lds_bytes<8, 2>()];
  RowsScaleEpilogue epi{a_scale, w_scale};
  gemm_core::rows32::run<I8Traits, 8, 2>(a, w_nk, K, epi, y, M, N, lds);
}
// ... and up to 128 rows: four row tiles, four waves (block = 256)
extern "C" __global__ void __launch_bounds__(256) mtrt_gemm_w8a8_nk_rows128(
    const int8_t* __restrict__ a, const int8_t* __restrict__ w_nk, const float* __restrict__ a_scale,
    const float* __restrict__ w_scale, uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N) {
  __shared__ __attribute__((aligned(16))) int8_t lds[gemm_core::rows32::lds_bytes<4, 4>()];
  RowsScaleEpilogue epi{a_scale, w_scale};
  gemm_core::rows32::run<I8Traits, 4, 4>(a, w_nk, K, epi, y, M, N, lds);
}

// Up to 32, 64 and 128 rows on fragment-order weights: the same kernels with the weight fragments straight from
// memory into registers.  (a [M,K] i8, w_frag, a_scale, w_scale, y, M, K, N) ; K % 128 == 0, a and w_frag 16-byte
// aligned; grid: any, block = 512 (rows32, rows64) / 256 (rows128).
extern "C" __global__ void __launch_bounds__(512) mtrt_gemm_w8a8_frag_rows32(
    const int8_t* __restrict__ a, const int8_t* __restrict__ w_frag, const float* __restrict__ a_scale,
    const float* __restrict__ w_scale, uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N) {
  __shared__ __attribute__((aligned(16))) int8_t lds[gemm_core::rows32::lds_bytes<8, 1, true>()];
  RowsScaleEpilogue epi{a_scale, w_scale};
  gemm_core::rows32::run<I8Traits, 8, 1, true>(a, w_frag, K, epi, y, M, N, lds);
}
extern "C" __global__ void __launch_bounds__(512) mtrt_gemm_w8a8_frag_rows64(
    const int8_t* __restrict__ a, const int8_t* __restrict__ w_frag, const float* __restrict__ a_scale,
    const float* __restrict__ w_scale, uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N) {
  __shared__ __attribute__((aligned(16))) int8_t lds[gemm_core::rows32::lds_bytes<8, 2, true>()];
  RowsScaleEpilogue epi{a_scale, w_scale};
  gemm_core::rows32::run<I8Traits, 8, 2, true>(a, w_frag, K, epi, y, M, N, lds);
}
extern "C" __global__ void __launch_bounds__(256) mtrt_gemm_w8a8_frag_rows128(
    const int8_t* __restrict__ a, const int8_t* __restrict__ w_frag, const float* __restrict__ a_scale,
    const float* __restrict__ w_scale, uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N) {
  __shared__ __attribute__((aligned(16))) int8_t lds[gemm_core::rows32::lds_bytes<4, 4, true>()];
  RowsScaleEpilogue epi{a_scale, w_scale};
  gemm_core::rows32::run<I8Traits, 4, 4, true>(a, w_frag, K, epi, y, M, N, lds);
}

// Any K and any operand alignment on the matrix cores, for the shapes the kernels above do not take (K not a
// multiple of 128, operands off 16-byte alignment, operands of 4 GiB and more): the 128 x 128 tile loop of
// gemm_core::edge.  (a [M,K] i8, w_nk [N,K] i8, a_scale [M] f32, w_scale [N] f32, y [M,N] f16, M, K, N)
// grid: any (tiles are dealt round-robin), block = 256.
struct EdgeScaleEpilogue {
  const float* a_scale;
  const float* w_scale;
  float as;
  __device__ __forceinline__ void row(int64_t row, bool valid) { as = valid ? a_scale[row] : 0.0f; }
  __device__ __forceinline__ uint32_t finish(int acc, int64_t col, bool valid) const {
    return f32_to_f16_bits((float(acc) * as) * (valid ? w_scale[col] : 0.0f));
  }
};

extern "C" __global__ void __launch_bounds__(256) mtrt_gemm_w8a8_nk_edge(
    const int8_t* __restrict__ a, const int8_t* __restrict__ w, const float* __restrict__ a_scale,
    const float* __restrict__ w_scale, uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N) {
  __shared__ __attribute__((aligned(16))) int8_t lds[gemm_core::edge::kLdsBytes];
  EdgeScaleEpilogue epi{a_scale, w_scale, 0.0f};
  gemm_core::edge::run<I8Traits>(a, w, K, epi, y, M, N, lds);
}

// Weight re-layout [K,N] -> [N,K], bytes.  64 x 64 tiles through LDS; both the global
// read and the global write are contiguous.  (w_kn, w_nk, K, N) grid = ceil(K/64)*ceil(N/64).
extern "C" __global__ void __launch_bounds__(256) mtrt_w8_prepack_kn_to_nk(const int8_t* __restrict__ w_kn,
                                                                         int8_t* __restrict__ w_nk, int64_t K, int64_t N) {
  __shared__ int8_t tile[64][65];
  const int64_t tiles_n = (N + 63) / 64;
  const int64_t k0 = int64_t(blockIdx.x / tiles_n) * 64, n0 = int64_t(blockIdx.x % tiles_n) * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int64_t k = k0 + ty + 4 * i, n = n0 + tx;
    if (k < K && n < N) tile[ty + 4 * i][tx] = w_kn[k * N + n];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int64_t n = n0 + ty + 4 * i, k = k0 + tx;
    if (k < K && n < N) w_nk[n * K + k] = tile[tx][ty + 4 * i];
  }
}

}  // namespace gemm_w8a8_cluster
