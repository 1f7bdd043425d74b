// W4A16 block-wise GEMM cluster for gfx950:
//     wd[k,n] = f16( f16(w_i4[k,n]) * s[k / block, n] )          (one f16 rounding)
//     y[m,n]  = f16( sum_k f32(a[m,k]) * f32(wd[k,n]) )            (f32 accumulation)
// the weight-only int4 form of the quantized Linear
// (tripy/nvtripy/frontend/module/linear.py:112-151, block dequantize as in
//  mlir-tensorrt/tensorrt/include/mlir-tensorrt-dialect/TensorRT/IR/TensorRTOps.td:3408-3445).
//
// Weights are program constants.  They arrive packed two per byte over the flattened
// [K,N] array (element 2i in the low nibble,
// mlir-tensorrt/tensorrt/lib/Target/TensorRTEncodingOpInterface/NetworkEncoder.cpp:552-595)
// and are re-laid ONCE by mtrt_w4_prepack into the order the matrix cores read:
//   for each tile of 32 columns and each block of 64 k, 64 lanes x 4 dwords, where
//   lane = 32*h + (n % 32) and dword j of that lane holds the 8 weights
//   k = 64*kb + 8*(2j + h) + [0..7] of column n.  Inside a dword nibble p (p < 4) is
//   weight 2p and nibble p + 4 is weight 2p + 1, each stored as (value + 8).
// A wave therefore loads 1 KiB of contiguous memory and every lane gets exactly its
// B-fragments for four v_mfma_f32_32x32x16_f16 steps; w & 0x000F000F isolates the pair
// (0, 1) in the two halves of a register, OR-ing 0x6400 into each half makes the f16
// numbers 1024 + (value + 8), a packed subtract of 1032 gives the exact integer value and
// a packed f16 multiply by the scale gives wd with the single rounding the program asks
// for; the pair (2, 3) is read where it sits (w & 0x00F000F0 under 0x5400: 64 + (value + 8),
// minus 72), the pairs (4, 5) and (6, 7) the same way from w >> 8.
//
// All kernels take the weight fragments straight from global memory into registers and
// dequantise them there; only the activations go through LDS (direct-to-LDS loads).
// Large M: 256 x 256 tiles, 4 waves of 256 x 64.  Medium M: 128 x 64 / 128 x 128 tiles so that the grid still fills
// the chip, 4 waves in two sets that split each K slice.
// Small M (<= 32): the GEMM is bound by reading the weights once.  One workgroup per
// 32 columns, its four waves split K, partial tiles are added through LDS at the end.
#include "gemm_core.hpp"

using namespace mtrt_dev;

namespace gemm_w4a16_cluster {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));

constexpr int BKH = 64;                              // k per slice (f16 elements): 128-byte LDS rows
constexpr int THREADS = 256;

__device__ __forceinline__ int lds_off(int row, int chunk) { return row * 128 + ((chunk ^ ((row >> 1) & 7)) << 4); }

union H2Bits { uint32_t u; h2 h; };

// One prepacked dword -> 8 dequantised f16 weights with a single shift: nibbles 0 and 2 are read in
// place under 0x6400 (1024 + u, minus 1032), nibbles 1 and 3 in place four bits higher under 0x5400
// (64 + 16 u / 16, minus 72); both differences are the exact integer, the multiply rounds once.
// The two masks (0x000F000F and 0x00F000F0) are held in vector registers: the and-or then is ONE
// instruction (it may name a single scalar or literal operand, and the exponent pattern is that one).
// dequant4 is half of it: dwords 2*part and 2*part + 1 of the chunk.
__device__ __forceinline__ void dequant4(uint32_t w, h2 scale2, int part, uint32_t mask_lo, uint32_t mask_hi, u4& out) {
  const h2 bias_lo = {(_Float16)1032.0f, (_Float16)1032.0f}, bias_hi = {(_Float16)72.0f, (_Float16)72.0f};
  const uint32_t v = part ? w >> 8 : w;
  H2Bits t0, t1;
  t0.u = (v & mask_lo) | 0x64006400u;
  t1.u = (v & mask_hi) | 0x54005400u;
  t0.h = (t0.h - bias_lo) * scale2;                    // exact integer, then one f16 rounding
  t1.h = (t1.h - bias_hi) * scale2;
  out[2 * part] = t0.u;
  out[2 * part + 1] = t1.u;
}
__device__ __forceinline__ u4 dequant8_in_place(uint32_t w, h2 scale2, uint32_t mask_lo, uint32_t mask_hi) {
  u4 out;
  dequant4(w, scale2, 0, mask_lo, mask_hi, out);
  dequant4(w, scale2, 1, mask_lo, mask_hi, out);
  return out;
}
__device__ __forceinline__ uint32_t nibble_pair_mask() {
  uint32_t m = 0x000F000Fu;
  __asm__ volatile("" : "+v"(m));                     // opaque to the compiler: stays in a vector register
  return m;
}

__device__ __forceinline__ h2 load_scale2(const uint16_t* __restrict__ scale, int64_t idx) {
  union { uint16_t u; _Float16 h; } c;
  c.u = scale[idx];
  h2 r = {c.h, c.h};
  return r;
}

// The entry points below have C linkage; they sit inside the namespace only so that
// its helper names do not meet those of the other clusters in the one-module build.

struct F16Traits {
  using Acc = v16f;
  static __device__ __forceinline__ Acc zero() {
    Acc z;
#pragma unroll
    for (int r = 0; r < 16; ++r) z[r] = 0.0f;
    return z;
  }
  static __device__ __forceinline__ Acc mfma(gemm_core::v4i a, gemm_core::v4i b, Acc c) {
    union { gemm_core::v4i i; v8h h; } ua, ub;
    ua.i = a; ub.i = b;
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(ua.h, ub.h, c, 0, 0, 0);
  }
  // The same with the accumulator held in ordinary vector registers.  With one wave per SIMD the compiler gives the
  // matrix instructions accumulation registers only (256 per lane); a tile with more than 256 accumulators keeps the
  // rest in the other half of the register file through these.  The compiler does not see inside: whoever reads such
  // an accumulator with another instruction waits for the matrix core first (settle_vgpr).
  static __device__ __forceinline__ void mfma_vgpr(gemm_core::v4i a, gemm_core::v4i b, Acc& c) {
    __asm__ volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void clear_vgpr(gemm_core::v4i a, gemm_core::v4i b, Acc& c) {
    __asm__ volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=v"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void settle_vgpr() { __asm__ volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }
};

struct PlainEpilogue {
  __device__ __forceinline__ void setup(int8_t*, int64_t, int64_t, int64_t, int64_t) {}
  __device__ __forceinline__ void row(int) {}
  template <int HC>
  __device__ __forceinline__ void columns(int) {}
  __device__ __forceinline__ void convert4(const v16f& acc, int q, int, uint32_t (&words)[2]) const {
#pragma unroll
    for (int e = 0; e < 4; e += 2) words[e >> 1] = f32x2_to_f16x2_bits(acc[4 * q + e], acc[4 * q + e + 1]);
  }
};

// ---- large M, weights straight into registers -------------------------------------------
// The prepacked stream is already in fragment order, so a wave can load the raw nibbles of
// its own columns (JT column tiles x 16 B per lane and slice) straight into registers and
// dequantise dword p of each into the B fragment of k-step p: the weights never touch LDS.
// LDS then carries the activations only (direct-to-LDS loads into a ring of 32 KiB
// stages, fetched two or four slices ahead), which takes the fragment reads, the panel stores and
// half of the direct-to-LDS traffic of the shared loop off the LDS port; waves that share
// columns (the row halves of a tile, the two sets that split a slice) dequantise the same weights,
// which is why the large tile gives each wave all 256 rows of its columns.
// Per k-step a wave issues IT x JT MFMAs in IT fenced chunks; each chunk also carries an A fragment
// read for the next k-step, its share of the next weights' dequantisation (13 VALU instructions per
// fragment) and, in k-step 0, its share of the direct-to-LDS loads.  Raw nibbles and scales of slice s+2 are
// fetched in the last k-step of slice s into the register set that k-step 2 finished with.
// D register sets = slices fetched ahead; KEEP: the waves use only part of each vector (see half)
template <int JT, int D, bool KEEP>
struct WeightRegs {
  const int8_t* wbase[JT];                           // slice 0 of each of this wave's 32-column tiles (uniform)
  const int8_t* scale;                               // as bytes (uniform)
  uint32_t wlane, scol[JT];                          // this lane's byte offsets inside a slice / inside a row of scales
  int64_t N;
  u4 raw[D][JT];
  uint32_t sc_bits[D][JT];
  uint32_t mask = nibble_pair_mask(), mask_hi = nibble_pair_mask() << 4;
  // tile0: first 32-column tile of this wave
  __device__ __forceinline__ void init(const uint32_t* wp, const uint16_t* sc, int64_t kblocks, int64_t n, int64_t tile0) {
    const int lane = threadIdx.x & 63;
    const int64_t last_tile = (n + 31) / 32 - 1;
    N = n;
    scale = reinterpret_cast<const int8_t*>(sc);
    wlane = uint32_t(lane) * 16;
#pragma unroll
    for (int j = 0; j < JT; ++j) {
      int64_t tile = tile0 + j;
      tile = tile < last_tile ? tile : last_tile;      // columns past N: some valid data, never stored
      int64_t col = tile * 32 + (lane & 31);
      col = col < n ? col : n - 1;
      wbase[j] = reinterpret_cast<const int8_t*>(wp) + tile * kblocks * 1024;
      scol[j] = uint32_t(col) * 2;
    }
  }
  // slice `slice` (its scales in row `srow`): scalar bases, 32-bit lane offsets kept opaque so that the loads take
  // them as they are (see DmaLoaderT::dma_at)
  template <int SET>
  __device__ __forceinline__ void fetch(uint32_t slice, const int8_t* srow_base) {
#pragma unroll
    for (int j = 0; j < JT; ++j) {
      __asm__ volatile("" : "+v"(wlane), "+v"(scol[j]));
      raw[SET][j] = *reinterpret_cast<const u4*>(wbase[j] + uint64_t(slice) * 1024 + wlane);
      sc_bits[SET][j] = *reinterpret_cast<const uint16_t*>(srow_base + scol[j]);
    }
  }
  template <int SET, int P>
  __device__ __forceinline__ void half(int j, int part, u4& frag) const {
    // Keeps all four dwords of the set allocated until here.  A wave that splits a slice with another
    // uses only two of them; the allocator would hand the other two out as scratch registers right
    // after the load was issued, and every write to such a register has to wait for the load first.
    if (KEEP) __asm__ volatile("" ::"v"(raw[SET][j]));
    H2Bits t;
    t.u = sc_bits[SET][j] * 0x00010001u;
    dequant4(raw[SET][j][P], t.h, part, mask, mask_hi, frag);
  }
};

// Shape of a workgroup: KW x MW x NWN waves.  MW x NWN waves tile the output, each 128 rows x
// 32*JT columns; with KW = 2 two such sets split every slice between them (k-steps KH and KH + 2
// of the four) and their accumulators are added at the end, which doubles the waves of a small
// tile without making the tile smaller.  A wave's own VALU, LDS and memory instructions do not
// overlap its MFMAs (each takes its issue cycles out of the MFMA stream), only another wave's
// do, so with the dequantisation in the loop two waves per SIMD are the faster shape.
// DEPTH: slices fetched ahead (weight register sets, and activation stages in flight); STAGES: activation
// stages in LDS, at least DEPTH + 1.  A tile with little work per slice needs the deeper ring: its loads
// must be issued a memory latency (about 2000 cycles under load) ahead, however few MFMA cycles a slice is.
// IT: 32-row tiles per wave (4: 128 rows; 8: 256 rows, one wave per SIMD owning a whole column of the tile).
// HS: 1 = the activation fragments of a whole k-step are read one k-step ahead (two sets of IT fragments);
// 2 = half a k-step ahead (two sets of IT / 2: the registers that a tile with more accumulators cannot spare).
template <int MW, int NWN, int JT, int KW, int DEPTH = 2, int STAGES = 4, int IT = 4, int HS = 1>
struct Shape {
  static constexpr int kMW = MW, kNWN = NWN, kJT = JT, kKW = KW, kDepth = DEPTH, kStages = STAGES, kIT = IT, kHS = HS;
  static_assert(HS == 1 || (HS == 2 && IT % 2 == 0), "fragments are read a whole or half a k-step ahead");
  static_assert(STAGES >= DEPTH + 1, "the stage being filled must not be one that is read");
  static constexpr int kSlots = MW * NWN, kWaves = KW * kSlots;
  static constexpr int kBM = 32 * IT * MW, kBN = 32 * JT * NWN;
  static constexpr int kStageBytes = kBM * 128;        // one slice of the activation panel
  static constexpr int kRingBytes = STAGES * kStageBytes;
  static constexpr int kOutBytes = kSlots * gemm_core::kOutWave + 2048;
  static constexpr int kSumBytes = KW == 2 ? kSlots * (32 * IT) * 32 * JT * 4 : 0;
  static constexpr int kLds = kRingBytes > kOutBytes ? (kRingBytes > kSumBytes ? kRingBytes : kSumBytes)
                                                     : (kOutBytes > kSumBytes ? kOutBytes : kSumBytes);
};

template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(gemm_core::IntC<I>{});
    static_for<I + 1, N>(f);
  }
}

template <class S, int KH, class Epilogue>
__device__ __forceinline__ void run_weight_regs(const int8_t* __restrict__ a, int64_t a_row_bytes,
                                                WeightRegs<S::kJT, S::kDepth, (S::kKW > 1)>& wr, uint32_t slices_per_block,
                                                Epilogue& epi, uint16_t* __restrict__ y, int64_t M, int64_t N, int64_t slices,
                                                int64_t m0, int64_t n0, int8_t* lds, int slot) {
  using namespace gemm_core;
  constexpr int JT = S::kJT, NWN = S::kNWN, KW = S::kKW, IT = S::kIT, G = (4 * IT * S::kMW) / S::kWaves, NK = 4 / KW;
  constexpr int D = S::kDepth, NS = S::kStages;
  // loads that may still be in flight when slice s+1 must have landed: those of the slices fetched
  // after it (G direct-to-LDS loads and 2 * JT register loads each) and this slice's own G
  constexpr int kFly = (D - 2) * (G + 2 * JT) + G;
  static_assert(kFly < 64, "wait counter range");
  static_assert((G < IT || G % IT == 0) && G <= 15, "direct-to-LDS loads per wave and slice, spread over the IT chunks");
  const int lane = threadIdx.x & 63;
  const int wm = slot / NWN;
  const int frow = lane & 31, fhalf = lane >> 5;

  v16f acc[IT][JT];
  // column tiles whose accumulators the compiler places (accumulation registers); those of the others are pinned to
  // ordinary vector registers (F16Traits::mfma_vgpr)
  constexpr int JA = IT * JT * 16 > 256 ? 256 / (IT * 16) : JT;

  const uint32_t nslices = uint32_t(slices), last = nslices - 1;
  DmaLoaderT<G> al;
  al.init(a, M, a_row_bytes, m0);
  // The slice fetched next, its row of scales and its position inside the block; moves on by one per slice until
  // it reaches the last slice (which is then fetched again into stages and registers that nobody reads).
  // (plain integer arithmetic instead of selects: it stays on the scalar unit)
  uint32_t fslice = 0, frem = 0;
  const int8_t* fsrow = wr.scale;
  const uint32_t scale_row_bytes = uint32_t(N) * 2;
  auto advance = [&]() {
    const uint32_t go = uint32_t(fslice - last) >> 31;                     // fslice < last
    fslice += go;
    frem += go;
    const uint32_t wrap = 1u - (uint32_t(frem - slices_per_block) >> 31);  // frem == slices_per_block (never above)
    frem &= wrap - 1u;
    fsrow += wrap * scale_row_bytes;
  };
  // Activation fragments: set P holds row tiles [0, IT) of the k-steps of parity P (HS == 1) or row tiles
  // [P * IT / 2, (P + 1) * IT / 2) of every k-step (HS == 2).  Weight fragments: set P for the k-steps of parity P.
  constexpr int HS = S::kHS, AN = IT / HS;
  v4i fa[2][AN];
  u4 fb[2][JT];
  // Fragment reads are issued as opaque instructions and waited for by count.  Left to the compiler every
  // k-step got one s_waitcnt lgkmcnt(0) placed right behind a read that had just been issued (its bookkeeping
  // of the in-order LDS counter gives up across the loop edge), so each k-step exposed one LDS round trip with
  // nothing else to issue.  The reads form one stream (chunk c of k-step t reads row tile c of k-step t+1); when
  // chunk c of k-step t+1 needs its fragment exactly IT - 1 younger reads are outstanding, whatever c is.
  // Row tile i of a wave sits i * 4096 bytes further; the swizzle depends on the lane and the k chunk only.
  const uint32_t lds_base = uint32_t(uintptr_t((lds_void_t*)lds));
  uint32_t a_lane[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) a_lane[p] = lds_base + uint32_t(lds_off(wm * (32 * IT) + frow, 2 * p + fhalf));
  auto read_a = [&](v4i& dst, uint32_t addr, auto tile) {
    constexpr int I = decltype(tile)::value;
    __asm__ volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(I * 4096) : "memory");
  };
  // the reads form one stream, AN chunks ahead of their use: AN - 1 younger ones may be outstanding
  auto landed_a = [&](v4i& frag) {
    __asm__ volatile("s_waitcnt lgkmcnt(%1)" : "+v"(frag) : "n"(AN - 1) : "memory");
  };
  auto stage_off = [&](uint32_t slice) { return uint32_t(slice % uint32_t(NS)) * uint32_t(S::kStageBytes); };
  auto stage = [&](uint32_t slice) { return lds + stage_off(slice); };

  auto prefetch = [&](auto d) {
    constexpr int DD = decltype(d)::value;
    const int8_t* src = al.slice_base(fslice);
#pragma unroll
    for (int g = 0; g < G; ++g) al.dma_at(src, stage(DD), g);
    wr.template fetch<DD>(fslice, fsrow);
    advance();
  };
  static_for<0, D>(prefetch);                          // register sets are named at compile time
  __builtin_amdgcn_sched_barrier(0);                   // (all of them issued here, none moved behind the barrier)
  // The accumulators are cleared by the matrix cores themselves (0 x 0 + 0) while the first loads are under way; written
  // as plain zeros the clearing (one register move per accumulator register) ends up behind the barrier, in front of
  // the loop, with nothing to overlap.
  {
    v4i none = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < IT; ++i)
#pragma unroll
      for (int j = 0; j < JT; ++j) {
        __asm__ volatile("" : "+v"(none));             // one MFMA per accumulator, not one result copied around
        if (j < JA) acc[i][j] = F16Traits::mfma(none, none, F16Traits::zero());
        else F16Traits::clear_vgpr(none, none, acc[i][j]);
      }
    __builtin_amdgcn_sched_barrier(0);
  }
  // The activations of slice 0 have landed; then meet the other waves.  Only the direct-to-LDS loads of the later slices
  // are counted as younger: the compiler may move register loads of the last sets behind this wait (it tracks those
  // itself), the direct-to-LDS loads stay where they are written, and slice 0's are the oldest of all.
  __builtin_amdgcn_s_waitcnt(0x0070 | (((D - 1) * G) & 15) | ((((D - 1) * G) >> 4) << 14));
  __asm__ volatile("s_barrier" ::: "memory");
  static_for<0, AN>([&](auto i) { read_a(fa[0][decltype(i)::value], a_lane[KH] + stage_off(0), i); });
#pragma unroll
  for (int j = 0; j < JT; ++j) {
    wr.template half<0, KH>(j, 0, fb[0][j]);
    wr.template half<0, KH>(j, 1, fb[0][j]);
  }

  // Step T (of NK) of a slice of parity PAR: MFMAs on `cur`, everything for this wave's next
  // k-step into `nxt`.  Four fenced chunks; chunk c multiplies row tile c and carries one A
  // fragment read, its share of the 2 * JT halves of the next weights' dequantisation and, in
  // step 0, G/4 direct-to-LDS loads.  Raw nibbles and scales of slice s+2 are fetched in the
  // last step into the register set that the step before finished with.
  // ca: LDS offset of the stage this k-step reads (HS == 2 only: its second half of row tiles is read during its first);
  // ra: of the stage the next k-step reads.
  auto kstep = [&](auto par, auto step, uint32_t ca, uint32_t ra, const int8_t* src, int8_t* nd) {
    constexpr int PAR = decltype(par)::value, T = decltype(step)::value;
    constexpr bool kLast = T == NK - 1;
    constexpr int NSET = kLast ? (PAR + 1) % D : PAR;  // register set and dword the next k-step's weights come from
    constexpr int NP = kLast ? KH : KH + (T + 1) * KW;
    constexpr int CUR = T % 2, NXT = 1 - CUR;          // weight fragment sets (and activation sets with HS == 1)
    const uint32_t raddr = a_lane[NP] + ra;
    const uint32_t caddr = a_lane[KH + T * KW] + ca;
    static_for<0, IT>([&](auto cc) {
      constexpr int c = decltype(cc)::value;
      constexpr int ASET = HS == 1 ? CUR : c / AN, AI = c % AN;
      landed_a(fa[ASET][AI]);
#pragma unroll
      for (int j = 0; j < JT; ++j) {
        if (j < JA) acc[c][j] = F16Traits::mfma(__builtin_bit_cast(v4i, fb[CUR][j]), fa[ASET][AI], acc[c][j]);
        else F16Traits::mfma_vgpr(__builtin_bit_cast(v4i, fb[CUR][j]), fa[ASET][AI], acc[c][j]);
      }
      if constexpr (HS == 1) read_a(fa[NXT][c], raddr, cc);
      else if constexpr (c < AN) read_a(fa[1][c], caddr, IntC<c + AN>{});          // row tile c + AN of this k-step
      else read_a(fa[0][c - AN], raddr, IntC<c - AN>{});                           // row tile c - AN of the next
#pragma unroll
      for (int u = 0; u < 2 * JT; ++u)
        if ((u * IT) / (2 * JT) == c) wr.template half<NSET, NP>(u >> 1, u & 1, fb[NXT][u >> 1]);
      if (T == 0) {
        if constexpr (G >= IT) {
#pragma unroll
          for (int g = 0; g < G / IT; ++g) al.dma_at(src, nd, c * (G / IT) + g);
        } else {
          if (c < G) al.dma_at(src, nd, c);
        }
      }
      if (kLast && c == 0) wr.template fetch<PAR>(fslice, fsrow);
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  auto slice_body = [&](auto par, uint32_t s) {
    const uint32_t pa = stage_off(s);
    const int8_t* src = al.slice_base(fslice);         // the slice fetched during this one: s + D, or the last
    int8_t* nd = stage(s + D);
    if (NK == 4) {
      kstep(par, IntC<0>{}, pa, pa, src, nd);
      kstep(par, IntC<1>{}, pa, pa, src, nd);
      kstep(par, IntC<NK == 4 ? 2 : 0>{}, pa, pa, src, nd);
    } else {
      kstep(par, IntC<0>{}, pa, pa, src, nd);
    }
    // slice s+1 and the registers of slice s+1 have landed; only younger loads may still fly
    // With a ring of at least D + 2 stages the fragment reads in flight belong to a stage that is not written before the
    // next barrier but one, and they need not be waited for here; with D + 1 stages the stage that the next slice's loads
    // fill is the one they read, so they are.
    constexpr int kLgkm = NS >= D + 2 ? 0x0F00 : 0x0000;
    __builtin_amdgcn_s_waitcnt(0x0070 | kLgkm | (kFly & 15) | ((kFly >> 4) << 14));   // vmcnt(kFly) [lgkmcnt(0)]
    __asm__ volatile("s_barrier" ::: "memory");
    kstep(par, IntC<NK - 1>{}, pa, stage_off(s + 1), src, nd);
    advance();
  };

  uint32_t s = 0;
  for (; s + D - 1 < nslices; s += D)                  // D slices per trip: one per register set, no branch inside
    static_for<0, D>([&](auto p) { slice_body(p, s + decltype(p)::value); });
  static_for<0, D - 1>([&](auto p) {
    if (s + decltype(p)::value < nslices) slice_body(p, s + decltype(p)::value);
  });
  __builtin_amdgcn_s_waitcnt(0x0070);                  // the surplus loads of the last slices have landed
  // ... and so have the surplus fragment reads: their registers stay allocated up to here
#pragma unroll
  for (int i = 0; i < AN; ++i) __asm__ volatile("s_waitcnt lgkmcnt(0)" ::"v"(fa[0][i]), "v"(fa[1][i]) : "memory");

  if (JA < JT) F16Traits::settle_vgpr();
  if (KW == 2) {                                       // second set hands its sums to the first through LDS
    __syncthreads();
    float* sum = reinterpret_cast<float*>(lds) + slot * ((32 * IT) * 32 * JT);
    if (KH == 1) {
#pragma unroll
      for (int i = 0; i < IT; ++i)
#pragma unroll
        for (int j = 0; j < JT; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q)
            *reinterpret_cast<f32x4*>(sum + (((i * JT + j) * 4 + q) * 64 + lane) * 4) =
                (f32x4){acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
    }
    __syncthreads();
    if (KH == 0) {
#pragma unroll
      for (int i = 0; i < IT; ++i)
#pragma unroll
        for (int j = 0; j < JT; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const f32x4 o = *reinterpret_cast<const f32x4*>(sum + (((i * JT + j) * 4 + q) * 64 + lane) * 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][j][4 * q + e] = acc[i][j][4 * q + e] + o[e];
          }
    }
  }
  write_tile<JT, NWN, S::kSlots>(acc, epi, y, M, N, m0, n0, lds, slot, KH == 0);
}

// Common body of the weight-in-register kernels: which tile, which wave does what.
template <class S>
__device__ __forceinline__ void weight_regs_kernel(const uint16_t* __restrict__ a, const uint32_t* __restrict__ wp,
                                                   const uint16_t* __restrict__ scale, uint16_t* __restrict__ y, int64_t M,
                                                   int64_t K, int64_t N, int64_t block, int8_t* lds) {
  int64_t tile_m, panel;
  // A slice of a 4-bit weight panel is a quarter of the bytes of an activation panel slice of the same
  // width: groups of four M tiles, eight panels at a time per XCD; every XCD the same number of tiles
  if (!gemm_core::tile_of_even(blockIdx.x, gridDim.x, (M + S::kBM - 1) / S::kBM, (N + S::kBN - 1) / S::kBN, 4, tile_m, panel)) return;
  const int64_t m0 = tile_m * S::kBM, n0 = panel * S::kBN;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int slot = wave % S::kSlots;
  WeightRegs<S::kJT, S::kDepth, (S::kKW > 1)> wr;
  wr.init(wp, scale, K / BKH, N, n0 / 32 + (slot % S::kNWN) * S::kJT);
  PlainEpilogue epi;
  const int8_t* ab = reinterpret_cast<const int8_t*>(a);
  const uint32_t spb = uint32_t(block / BKH);
  if (S::kKW == 1 || wave < S::kSlots) run_weight_regs<S, 0>(ab, 2 * K, wr, spb, epi, y, M, N, K / BKH, m0, n0, lds, slot);
  else run_weight_regs<S, S::kKW - 1>(ab, 2 * K, wr, spb, epi, y, M, N, K / BKH, m0, n0, lds, slot);
}

// (a [M,K] f16, w_prepacked, scale [K/block, N] f16, y [M,N] f16, M, K, N, block) ; K % 64 == 0, block % 64 == 0,
// a 16-byte aligned and below 4 GiB.  grid = 8 * ceil(ceil(N/256) * ceil(M/256) / 8), block = 256.
// Four waves, each a whole 256-row column of the tile (256 x 64, one wave per SIMD, 256 accumulator registers):
// a weight fragment is dequantised once per workgroup and a wave issues 16 MFMAs per k-step.  Against eight
// waves of 128 x 64 (every weight fragment dequantised by two waves) in one process: 343 -> 330 us at
// M = 4096, 94.9 -> 92.3 us at M = 1024, same bits.
using BigShape = Shape<1, 4, 2, 1, 2, 4, 8>;           // 256 x 256, 4 waves
extern "C" __global__ void __launch_bounds__(256, 1) mtrt_gemm_w4a16_t256x256(
    const uint16_t* __restrict__ a, const uint32_t* __restrict__ wp, const uint16_t* __restrict__ scale,
    uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N, int64_t block) {
  __shared__ __attribute__((aligned(16))) int8_t lds[BigShape::kLds];
  weight_regs_kernel<BigShape>(a, wp, scale, y, M, K, N, block, lds);
}
// 256 x 384 tiles: four waves of 256 x 96, 384 accumulator registers per lane, a third of them in ordinary vector
// registers (F16Traits::mfma_vgpr), activation fragments read half a k-step ahead.  A workgroup moves 44 KiB per
// slice for 384 MFMAs where the 256 x 256 tile moves 40 KiB for 256, and reads each activation fragment from LDS for
// three MFMAs instead of two.  Same argument list, grid = 8 * ceil(ceil(N/384) * ceil(M/256) / 8), block = 256.
// Against mtrt_gemm_w4a16_t256x256 in one process (K = 4096, N = 11008, the benchmark's data / zeros): M = 4096
// 298.4 -> 286.8 / 214.7 -> 207.1 us, M = 2048 (one round instead of two) 181 -> 145 / 141 -> 104, M = 8192 600 -> 571 /
// 430 -> 411; same bits.
using WideShape = Shape<1, 4, 3, 1, 2, 4, 8, 2>;       // 256 x 384, 4 waves
extern "C" __global__ void __launch_bounds__(256, 1) mtrt_gemm_w4a16_t256x384(
    const uint16_t* __restrict__ a, const uint32_t* __restrict__ wp, const uint16_t* __restrict__ scale,
    uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N, int64_t block) {
  __shared__ __attribute__((aligned(16))) int8_t lds[WideShape::kLds];
  weight_regs_kernel<WideShape>(a, wp, scale, y, M, K, N, block, lds);
}
// Medium M: 128 x 64 tiles so that the grid still fills the chip, two wave sets splitting each slice.
// Same argument list.  grid = 8 * ceil(ceil(N/64) * ceil(M/128) / 8), block = 256.
using MidShape = Shape<1, 2, 1, 2, 4, 5>;              // 128 x 64, 4 waves, four slices ahead (two workgroups share a CU's LDS)
extern "C" __global__ void __launch_bounds__(256) mtrt_gemm_w4a16_t128x64(
    const uint16_t* __restrict__ a, const uint32_t* __restrict__ wp, const uint16_t* __restrict__ scale,
    uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N, int64_t block) {
  __shared__ __attribute__((aligned(16))) int8_t lds[MidShape::kLds];
  weight_regs_kernel<MidShape>(a, wp, scale, y, M, K, N, block, lds);
}

// Medium M, wider: 128 x 128 tiles.  What a workgroup moves through its CU's L1 is dominated by the
// activation panel (16 KiB per slice against 2 KiB of weights per 64 columns), and the L1 is what bounds
// these launches, so the widest tile that still gives every compute unit a workgroup of its own is the
// fastest.
using MidWideShape = Shape<1, 4, 1, 2, 4, 8>;          // 128 x 128, 8 waves (two sets of four), four slices ahead, ring of eight stages (the stage of a slice is a mask away)
extern "C" __global__ void __launch_bounds__(512) mtrt_gemm_w4a16_t128x128(
    const uint16_t* __restrict__ a, const uint32_t* __restrict__ wp, const uint16_t* __restrict__ scale,
    uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N, int64_t block) {
  __shared__ __attribute__((aligned(16))) int8_t lds[MidWideShape::kLds];
  weight_regs_kernel<MidWideShape>(a, wp, scale, y, M, K, N, block, lds);
}

// Medium M, twice as wide: 128 x 256 tiles, the same eight waves with two column tiles each.  An activation fragment
// read from LDS serves two MFMAs and the activation panel is fetched for half as many workgroups; a slice takes 0.48 us
// against 0.37 us for twice the MFMAs, so a full round of these tiles costs 1.9 rounds of the 128 x 128 ones: ahead where
// it saves a round (K = 4096, N = 11008: M = 512 56.9 -> 51.3 us, M = 300 53.8 -> 47.5; K = N = 8192, M = 1024 124.9 -> 115.9),
// behind where the narrower tile fits one round anyway (M = 256: 43.6 against 27.3 us).
using MidWide2Shape = Shape<1, 4, 2, 2, 4, 8>;         // 128 x 256, 8 waves (two sets of four), four slices ahead
extern "C" __global__ void __launch_bounds__(512) mtrt_gemm_w4a16_t128x256(
    const uint16_t* __restrict__ a, const uint32_t* __restrict__ wp, const uint16_t* __restrict__ scale,
    uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N, int64_t block) {
  __shared__ __attribute__((aligned(16))) int8_t lds[MidWide2Shape::kLds];
  weight_regs_kernel<MidWide2Shape>(a, wp, scale, y, M, K, N, block, lds);
}

// Small M (<= 32): one workgroup per 32 columns, four waves split K.
// G: groups of 8 activation rows kept per stage (M <= 8 * G); WAVES: waves that split K;
// JT: column tiles of the workgroup (blockIdx.x, blockIdx.x + gridDim.x), sharing the activations.
template <int G, int WAVES, int JT>
__device__ __forceinline__ void skinny(const uint16_t* __restrict__ a, const uint32_t* __restrict__ wp,
                                       const uint16_t* __restrict__ scale, uint16_t* __restrict__ y, int64_t M, int64_t K,
                                       int64_t N, int64_t block, int8_t* lds) {
  // Per wave a ring of four stages (8 * G rows x 64 k of activations each), filled by
  // direct-to-LDS loads three slices ahead: a fragment read straight from global memory would
  // touch 64 different cache lines per instruction (32 rows 8 KiB apart), the ring is filled
  // with whole 128-byte row segments.  The waves never touch each other's ring: no barriers.
  constexpr int kStages = 4, kStageBytes = 8 * G * 128;
  constexpr int kLoads = G + 2 * JT;                 // memory instructions per slice and wave
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int frow = lane & 31, fhalf = lane >> 5;
  const int64_t kblocks = K / BKH;
  const int64_t kb0 = kblocks * wave / WAVES, kb1 = kblocks * (wave + 1) / WAVES;
  const uint32_t slices_per_block = uint32_t(block / BKH);
  int64_t tile[JT], col[JT];
  const u4* bp[JT];
#pragma unroll
  for (int j = 0; j < JT; ++j) {
    tile[j] = blockIdx.x + int64_t(j) * gridDim.x;
    col[j] = tile[j] * 32 + frow;
    col[j] = col[j] < N ? col[j] : N - 1;            // columns past N: the last column's scales, never stored
    bp[j] = reinterpret_cast<const u4*>(wp) + (tile[j] * kblocks) * 64 + lane;
  }
  int8_t* ring = lds + wave * (kStages * kStageBytes);

  // direct-to-LDS load g (of G) of a slice: rows 8g .. 8g+7, lane l <-> (row l >> 3, LDS chunk l & 7)
  uint32_t aoff[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const int lrow = g * 8 + (lane >> 3);
    const int64_t row = lrow < M ? lrow : M - 1;     // rows past M repeat the last row; never stored
    aoff[g] = uint32_t(row * K * 2 + (((lane & 7) ^ ((lrow >> 1) & 7)) << 4));
  }
  const int8_t* abase = reinterpret_cast<const int8_t*>(a);
  struct Slice {
    u4 w[JT];
    uint32_t sc[JT];
  };
  // everything slice kb needs from memory: G + 2 JT loads, always, so that the waits can count
  auto fetch = [&](int64_t kb, int64_t clamp, Slice& dst) {
    kb = kb < clamp ? kb : clamp;
    int8_t* st = ring + int(kb & (kStages - 1)) * kStageBytes;
#pragma unroll
    for (int g = 0; g < G; ++g)
      __builtin_amdgcn_global_load_lds((gemm_core::global_void_t*)(abase + kb * (BKH * 2) + aoff[g]),
                                       (gemm_core::lds_void_t*)(st + g * 1024), 16, 0, 0);
    // Register loads issued as opaque instructions: the compiler's own wait-count bookkeeping
    // gives up on loads carried around a loop and drains everything (vmcnt(0)) before their first
    // use, which would leave nothing in flight.  The waits are placed by hand in `landed`.
#pragma unroll
    for (int j = 0; j < JT; ++j) {
      const u4* wsrc = bp[j] + kb * 64;
      const uint16_t* ssrc = scale + int64_t(uint32_t(kb) / slices_per_block) * N + col[j];
      __asm__ volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(dst.w[j]) : "v"(wsrc) : "memory");
      __asm__ volatile("global_load_ushort %0, %1, off" : "=v"(dst.sc[j]) : "v"(ssrc) : "memory");
    }
  };
  // ties the registers of a slice to the wait, so that no use can be scheduled in front of it:
  // four slices issued, the loads of three may fly -> those of the oldest slice have landed
  auto landed = [&](Slice& sl) {
#pragma unroll
    for (int j = 0; j < JT; ++j)
      __asm__ volatile("s_waitcnt vmcnt(%2)" : "+v"(sl.w[j]), "+v"(sl.sc[j]) : "n"(3 * kLoads) : "memory");
  };
  auto landed_all = [&](Slice& sl) {
#pragma unroll
    for (int j = 0; j < JT; ++j) __asm__ volatile("s_waitcnt vmcnt(0)" : "+v"(sl.w[j]), "+v"(sl.sc[j])::"memory");
  };

  v16f acc[JT];
#pragma unroll
  for (int j = 0; j < JT; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.0f;
  const uint32_t mask = nibble_pair_mask(), mask_hi = mask << 4;
  auto multiply = [&](int64_t kb, const Slice& sl) {
    const int8_t* st = ring + int(kb & (kStages - 1)) * kStageBytes;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const int arow = frow < 8 * G ? frow : 8 * G - 1;   // rows past the ring: any valid data, never stored
      const v8h fa = *reinterpret_cast<const v8h*>(st + gemm_core::lds_off(arow, 2 * ks + fhalf));
#pragma unroll
      for (int j = 0; j < JT; ++j) {
        H2Bits sp;
        sp.u = sl.sc[j] * 0x00010001u;
        union { u4 u; v8h h; } fb;
        fb.u = dequant8_in_place(sl.w[j][ks], sp.h, mask, mask_hi);
        acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa, fb.h, acc[j], 0, 0, 0);
      }
    }
  };

  // Main part: groups of four slices with four register sets, so that nothing is copied (a copy
  // would have to wait for the load) and the loop has no branch; three slices stay in flight.
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
  float (*partial)[16][64] = reinterpret_cast<float (*)[16][64]>(lds);
#pragma unroll
  for (int j = 0; j < JT; ++j) {
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 16; ++r) partial[wave][r][lane] = acc[j][r];
    __syncthreads();
    for (int e = threadIdx.x; e < 16 * 64; e += 64 * WAVES) {
      const int r = e >> 6, l = e & 63;
      float v = partial[0][r][l];
#pragma unroll
      for (int w = 1; w < WAVES; ++w) v = v + partial[w][r][l];
      const int64_t row = (r >> 2) * 8 + (l >> 5) * 4 + (r & 3);
      const int64_t c = tile[j] * 32 + (l & 31);
      if (row < M && c < N) y[row * N + c] = uint16_t(f32_to_f16_bits(v));
    }
  }
}

// The grid is one workgroup per column tile, or, while that would leave some compute units with two
// workgroups and the rest with one (tiles between one and two times the compute units), one workgroup
// per compute unit: workgroup g then also takes tile g + gridDim.x if there is one, and reads the
// activations once for both.
template <int G>
__device__ __forceinline__ void skinny_tiles(const uint16_t* __restrict__ a, const uint32_t* __restrict__ wp,
                                             const uint16_t* __restrict__ scale, uint16_t* __restrict__ y, int64_t M,
                                             int64_t K, int64_t N, int64_t block, int8_t* lds) {
  const int64_t tiles = (N + 31) / 32;
  if (int64_t(blockIdx.x) + gridDim.x < tiles)
    skinny<G, 4, 2>(a, wp, scale, y, M, K, N, block, lds);
  else
    skinny<G, 4, 1>(a, wp, scale, y, M, K, N, block, lds);
}

// M <= 16: half the activation rows per stage (8 waves splitting K were no faster than 4).
extern "C" __global__ void __launch_bounds__(256) mtrt_gemm_w4a16_skinny16(
    const uint16_t* __restrict__ a, const uint32_t* __restrict__ wp, const uint16_t* __restrict__ scale,
    uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N, int64_t block) {
  __shared__ __attribute__((aligned(16))) int8_t lds[4 * 4 * 2 * 1024];
  skinny_tiles<2>(a, wp, scale, y, M, K, N, block, lds);
}
// M <= 32: 4 waves split K.
extern "C" __global__ void __launch_bounds__(256) mtrt_gemm_w4a16_skinny(
    const uint16_t* __restrict__ a, const uint32_t* __restrict__ wp, const uint16_t* __restrict__ scale,
    uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N, int64_t block) {
  __shared__ __attribute__((aligned(16))) int8_t lds[4 * 4 * 4 * 1024];
  skinny_tiles<4>(a, wp, scale, y, M, K, N, block, lds);
}

// ---- M <= 16: one strip of columns per compute unit --------------------------------------------------
// At this size the launch is bound by what each compute unit's L1 takes in: its share of the weights plus ALL of
// the activations (16 rows x K).  One workgroup per 32-column tile leaves 344 workgroups on 256 compute units at
// N = 11008, and the 88 units that hold two set the time.  Here the grid is one workgroup per compute unit, each
// owning a contiguous strip of 16-column tiles (688 tiles -> 2 or 3 per workgroup, at most 48 of the ideal 43
// columns) over ALL of K: no second round, no partial sums across workgroups.
// 16-column tiles need v_mfma_f32_16x16x32_f16 (lane l: column l % 16, k group l / 16, 8 consecutive k), so this
// kernel reads the weights from a second re-layout made by mtrt_w4_prepack_strips:
//   for each tile of 16 columns and each block of 128 k, 64 lanes x 4 dwords; dword j of lane l holds the 8 weights
//   k = 128*kb + 32*j + 8*(l / 16) + [0..7] of column 16*tile + l % 16, nibbles ordered as in the 32-column layout.
// The four waves of a workgroup split K; each keeps its own four-stage ring of activation slices (16 rows x 128 k,
// whole 256-byte row segments by direct-to-LDS loads, 16-byte chunks XOR-swizzled by the row so that the fragment
// reads are conflict-free) and never touches another wave's ring: no barriers until the partial tiles are added
// through LDS at the end.
typedef float v4f __attribute__((ext_vector_type(4)));

template <int WAVES, int JT>
__device__ __forceinline__ void strips_chunk(const uint16_t* __restrict__ a, const uint32_t* __restrict__ ws,
                                             const uint16_t* __restrict__ scale, uint16_t* __restrict__ y, int64_t M,
                                             int64_t K, int64_t N, int64_t block, int64_t tile0, int8_t* lds) {
  constexpr int kStages = 4, kStageBytes = 16 * 256;   // 16 rows x 128 k of f16
  constexpr int kLoads = 4 + 2 * JT;                   // memory instructions per slice and wave
  static_assert(3 * kLoads < 64, "wait counter range");
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int fcol = lane & 15, fgrp = lane >> 4;
  const int64_t kblocks = K / 128;
  const int64_t kb0 = kblocks * wave / WAVES, kb1 = kblocks * (wave + 1) / WAVES;
  const uint32_t blocks_per_scale = uint32_t(block / 128);
  int64_t col[JT];
  const u4* bp[JT];
#pragma unroll
  for (int j = 0; j < JT; ++j) {
    col[j] = (tile0 + j) * 16 + fcol;
    col[j] = col[j] < N ? col[j] : N - 1;              // columns past N: the last column's scales, never stored
    bp[j] = reinterpret_cast<const u4*>(ws) + ((tile0 + j) * kblocks) * 64 + lane;
  }
  int8_t* ring = lds + wave * (kStages * kStageBytes);

  // direct-to-LDS load g (of 4) of a slice: rows 4g .. 4g+3; lane l <-> (row 4g + l / 16, LDS chunk position l % 16),
  // which holds chunk (l % 16) ^ row of that row's 256 bytes
  uint32_t aoff[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const int lrow = 4 * g + (lane >> 4);
    const int64_t row = lrow < M ? lrow : M - 1;       // rows past M repeat the last row; never stored
    aoff[g] = uint32_t(row * K * 2 + (((lane & 15) ^ lrow) << 4));
  }
  const int8_t* abase = reinterpret_cast<const int8_t*>(a);
  struct Slice {
    u4 w[JT];
    uint32_t sc[JT];
  };
  auto fetch = [&](int64_t kb, int64_t clamp, Slice& dst) {
    kb = kb < clamp ? kb : clamp;
    int8_t* st = ring + int(kb & (kStages - 1)) * kStageBytes;
#pragma unroll
    for (int g = 0; g < 4; ++g)
      __builtin_amdgcn_global_load_lds((gemm_core::global_void_t*)(abase + kb * 256 + aoff[g]),
                                       (gemm_core::lds_void_t*)(st + g * 1024), 16, 0, 0);
    // opaque register loads, waits placed by hand (see `skinny`)
#pragma unroll
    for (int j = 0; j < JT; ++j) {
      const u4* wsrc = bp[j] + kb * 64;
      const uint16_t* ssrc = scale + int64_t(uint32_t(kb) / blocks_per_scale) * N + col[j];
      __asm__ volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(dst.w[j]) : "v"(wsrc) : "memory");
      __asm__ volatile("global_load_ushort %0, %1, off" : "=v"(dst.sc[j]) : "v"(ssrc) : "memory");
    }
  };
  auto landed = [&](Slice& sl) {
#pragma unroll
    for (int j = 0; j < JT; ++j)
      __asm__ volatile("s_waitcnt vmcnt(%2)" : "+v"(sl.w[j]), "+v"(sl.sc[j]) : "n"(3 * kLoads) : "memory");
  };
  auto landed_all = [&](Slice& sl) {
#pragma unroll
    for (int j = 0; j < JT; ++j) __asm__ volatile("s_waitcnt vmcnt(0)" : "+v"(sl.w[j]), "+v"(sl.sc[j])::"memory");
  };

  v4f acc[JT];
#pragma unroll
  for (int j = 0; j < JT; ++j) acc[j] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
  const uint32_t mask = nibble_pair_mask(), mask_hi = mask << 4;
  auto multiply = [&](int64_t kb, const Slice& sl) {
    const int8_t* st = ring + int(kb & (kStages - 1)) * kStageBytes;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const v8h fa = *reinterpret_cast<const v8h*>(st + fcol * 256 + (((4 * ks + fgrp) ^ fcol) << 4));
#pragma unroll
      for (int j = 0; j < JT; ++j) {
        H2Bits sp;
        sp.u = sl.sc[j] * 0x00010001u;
        union { u4 u; v8h h; } fb;
        fb.u = dequant8_in_place(sl.w[j][ks], sp.h, mask, mask_hi);
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa, fb.h, acc[j], 0, 0, 0);
      }
    }
  };

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
  // partial tiles of the waves meet in LDS: [wave][tile][register][lane]
  float* partial = reinterpret_cast<float*>(lds);
  __syncthreads();
#pragma unroll
  for (int j = 0; j < JT; ++j)
#pragma unroll
    for (int r = 0; r < 4; ++r) partial[((wave * JT + j) * 4 + r) * 64 + lane] = acc[j][r];
  __syncthreads();
  for (int e = threadIdx.x; e < JT * 4 * 64; e += 64 * WAVES) {
    const int l = e & 63, r = (e >> 6) & 3, j = e >> 8;
    float v = partial[((0 * JT + j) * 4 + r) * 64 + l];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) v = v + partial[((w * JT + j) * 4 + r) * 64 + l];
    const int64_t row = 4 * (l >> 4) + r;
    const int64_t c = (tile0 + j) * 16 + (l & 15);
    if (row < M && c < N) y[row * N + c] = uint16_t(f32_to_f16_bits(v));
  }
  __syncthreads();                                     // the next chunk of this workgroup reuses the LDS
}

// (a [M,K] f16, strip-order weights, scale [K/block, N] f16, y [M,N] f16, M <= 16, K % 128 == 0, N, block % 128 == 0)
// grid = min(compute units, ceil(N / 16)), block = 256: workgroup g owns tiles / grid consecutive 16-column tiles (the first
// tiles % grid workgroups one more), three at a time.
// Four waves, one per SIMD.  Measured on M = 16, N = 11008, K = 4096 (rocprofv3 kernel durations): 2 / 4 / 8 waves take
// 12.7 / 9.6 / 10.7 us; more than one workgroup per compute unit (grids of 344, 512, 688) 11.5-12.6 us.  In-kernel
// timestamps of the four-wave form: 1.3 us until the loads are issued, first slice landed at 3.9 us, K loop done at
// 10.4 us (1600 cycles per slice against some 800 of issue for 175 dequantisation instructions and 12 MFMAs), so what
// is left is the dequantisation on one wave per SIMD and the 4 us before the first data; with eight waves the loop
// shortens to 4.9 us but the first data arrives later by as much.
constexpr int kStripWaves = 4;
extern "C" __global__ void __launch_bounds__(64 * kStripWaves) mtrt_gemm_w4a16_strips16(
    const uint16_t* __restrict__ a, const uint32_t* __restrict__ ws, const uint16_t* __restrict__ scale,
    uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N, int64_t block) {
  __shared__ __attribute__((aligned(16))) int8_t lds[kStripWaves * 4 * 4096];
  // tiles / grid tiles each, the first tiles % grid workgroups one more (32-bit arithmetic: as 64-bit divisions this was
  // a microsecond of scalar instructions in front of the first load)
  const uint32_t tiles = uint32_t((N + 15) / 16), grid = gridDim.x, b = blockIdx.x;
  const uint32_t per = tiles / grid, rem = tiles - per * grid;
  const int64_t t0 = int64_t(b * per + (b < rem ? b : rem)), t1 = t0 + per + (b < rem ? 1 : 0);
  for (int64_t t = t0; t < t1; t += 3) {
    const int64_t left = t1 - t;
    if (left >= 3) strips_chunk<kStripWaves, 3>(a, ws, scale, y, M, K, N, block, t, lds);
    else if (left == 2) strips_chunk<kStripWaves, 2>(a, ws, scale, y, M, K, N, block, t, lds);
    else strips_chunk<kStripWaves, 1>(a, ws, scale, y, M, K, N, block, t, lds);
  }
}

// Re-layout for mtrt_gemm_w4a16_strips16: packed [K,N] nibbles -> strip order (above).  One thread per output dword.
// (w_kn_packed, ws, K, N) ; K % 128 == 0.
extern "C" __global__ void __launch_bounds__(256) mtrt_w4_prepack_strips(const uint8_t* __restrict__ w_kn_packed,
                                                                       uint32_t* __restrict__ ws, int64_t K, int64_t N) {
  const int64_t kblocks = K / 128;
  const int64_t ntiles = (N + 15) / 16;
  const int64_t total = ntiles * kblocks * 256;
  for (int64_t d = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; d < total; d += int64_t(gridDim.x) * blockDim.x) {
    const int j = int(d & 3), lane = int((d >> 2) & 63);
    const int64_t kb = (d >> 8) % kblocks, tile = (d >> 8) / kblocks;
    const int64_t n = tile * 16 + (lane & 15);
    const int64_t k0 = kb * 128 + 32 * j + 8 * (lane >> 4);
    uint32_t w = 0;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      uint32_t nib = 0;                                 // columns past N: value 0
      if (n < N) {
        const int64_t i = (k0 + q) * N + n;
        const uint32_t byte = w_kn_packed[i >> 1];
        nib = (i & 1) ? (byte >> 4) : (byte & 0xFu);
      }
      const uint32_t u = (nib ^ 8u) & 0xFu;             // value + 8
      const int pos = (q & 1) ? (q >> 1) + 4 : (q >> 1);
      w |= u << (4 * pos);
    }
    ws[d] = w;
  }
}

// Any K, N and block on the matrix cores, reading the ORIGINAL packed [K,N] nibbles: for shapes the kernels above do
// not take (blocks that are not multiples of 64, K that is not, no re-laid weights, operands off alignment).  The
// 128 x 128 tile loop of gemm_core::edge with the weight stage produced here: a k-step of 64 rows x 128 columns of
// nibbles (65 bytes a row when a row starts on an odd nibble) goes through registers into a raw LDS stage of 17
// dwords per row; then every lane takes one k row of the step and dequantises eight columns at a time (one dword of
// nibbles -> f32, times the eight scales of the row's block fetched a k-step ahead, one rounding to f16 each) into
// 16-bit pieces of the [column][k] stage the fragments are read from.  Rows at and past K and columns at and past
// N become zeros without touching their scales.
// (a [M,K] f16, w_kn_packed, scale [K/block, N] f16, y [M,N] f16, M, K, N, block) grid: any, block = 256.
namespace edge4 {
constexpr int kRawRow = 68;                            // bytes of a raw row: 17 dwords cover 65 bytes from any byte offset
constexpr int kRawBytes = 64 * kRawRow;
typedef uint32_t u32_bytes __attribute__((aligned(1)));

struct HalfEpilogue {
  __device__ __forceinline__ void row(int64_t, bool) {}
  __device__ __forceinline__ uint32_t finish(float acc, int64_t, bool) const { return f32_to_f16_bits(acc); }
};

// dword `dw` of the raw row of k: the bytes holding nibbles (k, n0 ...) onwards; zeros past K.  The last bytes of the
// weights can end inside a dword: that dword is zero here and read byte by byte by finish_raw.
__device__ __forceinline__ uint32_t load_raw(const uint8_t* __restrict__ w, int64_t k, int64_t K, int64_t N, int64_t n0, int dw,
                                             int64_t total_bytes) {
  const int64_t at = ((k * N + n0) >> 1) + 4 * dw;
  uint32_t v = 0;
  if (k < K && at + 4 <= total_bytes) v = *reinterpret_cast<const u32_bytes*>(w + at);
  return v;
}
__device__ __forceinline__ uint32_t finish_raw(uint32_t v, const uint8_t* __restrict__ w, int64_t k, int64_t K, int64_t N, int64_t n0,
                                               int dw, int64_t total_bytes) {
  const int64_t at = ((k * N + n0) >> 1) + 4 * dw;
  if (k >= K || at + 4 <= total_bytes) return v;
#pragma unroll 1
  for (int b = 0; b < 4; ++b)
    if (at + b < total_bytes) v |= uint32_t(w[at + b]) << (8 * b);
  return v;
}
// the five dwords of the raw stage a lane moves per k-step (17 per row, 64 rows from k0 on)
__device__ __forceinline__ void load_raws(uint32_t (&r)[5], const uint8_t* __restrict__ w, int64_t k0, int64_t K, int64_t N, int64_t n0,
                                          int64_t total_bytes) {
#pragma unroll
  for (int i = 0; i < 5; ++i) {
    const int idx = threadIdx.x + 256 * i;
    r[i] = idx < 64 * 17 ? load_raw(w, k0 + idx / 17, K, N, n0, idx % 17, total_bytes) : 0u;
  }
  // only the rows next to the end of the weights can have such a dword (the same test for the whole workgroup)
  const int64_t k_hi = k0 + 63 < K ? k0 + 63 : K - 1;
  if (((k_hi * N + n0) >> 1) + 4 * 17 > total_bytes) {
#pragma unroll
    for (int i = 0; i < 5; ++i) {
      const int idx = threadIdx.x + 256 * i;
      if (idx < 64 * 17) r[i] = finish_raw(r[i], w, k0 + idx / 17, K, N, n0, idx % 17, total_bytes);
    }
  }
}

// the f16 scales of columns n .. n + 7 in the block of row k, as four words of two; zeros where the element does not
// exist.  Fetched a k-step ahead and widened only where they are used, so that the load is not waited for where it
// is issued; all lanes of a wave whose rows share a block read the same 16 bytes.
typedef u32x4 u32x4_halves __attribute__((aligned(2)));
__device__ __forceinline__ u32x4 load_scales8(const uint16_t* __restrict__ scale, int64_t k, int64_t K, int64_t N, int64_t n, uint32_t blk) {
  u32x4 v = {0u, 0u, 0u, 0u};
  if (k >= K || n >= N) return v;
  const uint16_t* p = scale + int64_t(uint32_t(k) / blk) * N + n;
  if (n + 8 <= N) return *reinterpret_cast<const u32x4_halves*>(p);
#pragma unroll
  for (int j = 0; j < 8; ++j)
    if (n + j < N) v[j >> 1] |= uint32_t(p[j]) << (16 * (j & 1));
  return v;
}
}  // namespace edge4

extern "C" __global__ void __launch_bounds__(256) mtrt_gemm_w4a16_edge(
    const uint16_t* __restrict__ a, const uint8_t* __restrict__ w_kn_packed, const uint16_t* __restrict__ scale,
    uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N, int64_t block) {
  namespace ge = gemm_core::edge;
  using namespace edge4;
  __shared__ __attribute__((aligned(16))) int8_t lds[ge::kLdsBytes + kRawBytes];
  int8_t* sa = lds;
  int8_t* sb = lds + ge::kTile * ge::kPitch;
  uint8_t* raw = reinterpret_cast<uint8_t*>(lds + ge::kLdsBytes);
  const int8_t* a8 = reinterpret_cast<const int8_t*>(a);
  const int64_t row_bytes = K * 2, total_bytes = (K * N + 1) >> 1;
  const int64_t tiles_m = (M + ge::kTile - 1) / ge::kTile, tiles_n = (N + ge::kTile - 1) / ge::kTile;
  const int64_t steps = (K + 63) / 64;
  const int crow = threadIdx.x >> 3, ccol = (threadIdx.x & 7) * 16;
  const int drow = threadIdx.x & 63, dwave = threadIdx.x >> 6;       // dequantise: k row of the step, column groups 4 dwave + i
  const uint32_t blk = uint32_t(block);
  HalfEpilogue epi;
  for (int64_t tile = blockIdx.x; tile < tiles_m * tiles_n; tile += gridDim.x) {
    const int64_t m0 = (tile % tiles_m) * ge::kTile, n0 = (tile / tiles_m) * ge::kTile;
    v16f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = F16Traits::zero();
    u32x4 ra[4];
    uint32_t rw[5];
    u32x4 rs[4];                                       // the eight scales (f16 bits) of each of the lane's four column groups
    ge::load_chunks(ra, a8, m0, M, row_bytes, ccol, steps == 1);
    load_raws(rw, w_kn_packed, 0, K, N, n0, total_bytes);
#pragma unroll
    for (int i = 0; i < 4; ++i) rs[i] = load_scales8(scale, drow, K, N, n0 + (4 * dwave + i) * 8, blk);
    for (int64_t s = 0; s < steps; ++s) {
      __syncthreads();                                 // the previous k-step's (or tile's) LDS reads are done
#pragma unroll
      for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(sa + (crow + 32 * i) * ge::kPitch + ccol) = ra[i];
#pragma unroll
      for (int i = 0; i < 5; ++i) {
        const int idx = threadIdx.x + 256 * i;
        if (idx < 64 * 17) *reinterpret_cast<uint32_t*>(raw + 4 * idx) = rw[i];
      }
      __syncthreads();
      {
        // lane = k row of the step: its eight nibbles of a column group are one aligned dword of the raw row (plus
        // the next byte when the row starts on an odd nibble), its stores are 16-bit pieces of eight columns' rows of
        // the [column][k] stage, 64 lanes side by side in k.  Rows at and past K hold zero nibbles and get zero
        // scales, columns at and past N zero scales.
        const uint8_t* rrow = raw + drow * kRawRow;
        const uint32_t shift = 4u * uint32_t(((s * 64 + drow) & N) & 1);   // n0 is even: the row starts at nibble (k N) mod 2
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int cg = 4 * dwave + i;
          const uint32_t lo = *reinterpret_cast<const uint32_t*>(rrow + 4 * cg), hi = rrow[4 * cg + 4];
          const uint32_t nibbles = uint32_t(((uint64_t(hi) << 32) | lo) >> shift);
          int8_t* dst = sb + (cg * 8) * ge::kPitch + drow * 2;
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float sc = f16_bits_to_f32((rs[i][j >> 1] >> (16 * (j & 1))) & 0xFFFFu);
            const uint32_t bits = f32_to_f16_bits(float(int(nibbles << (28 - 4 * j)) >> 28) * sc);
            *reinterpret_cast<uint16_t*>(dst + j * ge::kPitch) = uint16_t(bits);
          }
        }
      }
      __syncthreads();
      if (s + 1 < steps) {
        ge::load_chunks(ra, a8, m0, M, row_bytes, (s + 1) * ge::kStep + ccol, s + 2 == steps);
        load_raws(rw, w_kn_packed, (s + 1) * 64, K, N, n0, total_bytes);
#pragma unroll
        for (int i = 0; i < 4; ++i) rs[i] = load_scales8(scale, (s + 1) * 64 + drow, K, N, n0 + (4 * dwave + i) * 8, blk);
      }
      ge::multiply_stage<F16Traits>(acc, sa, sb);
    }
    ge::write_tile(acc, epi, y, M, N, m0, n0, lds);
  }
}

// Any shape: one output per lane, reading the ORIGINAL packed [K,N] nibbles; not a fast path.
extern "C" __global__ void __launch_bounds__(256) mtrt_gemm_w4a16_any(
    const uint16_t* __restrict__ a, const uint8_t* __restrict__ w_kn_packed, const uint16_t* __restrict__ scale,
    uint16_t* __restrict__ y, int64_t M, int64_t K, int64_t N, int64_t block) {
  const int64_t total = M * N;
  for (int64_t e = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; e < total; e += int64_t(gridDim.x) * blockDim.x) {
    const int64_t m = e / N, n = e - m * N;
    float acc = 0.0f;
    for (int64_t k = 0; k < K; ++k) {
      const int64_t i = k * N + n;
      const uint32_t byte = w_kn_packed[i >> 1];
      const uint32_t nib = (i & 1) ? (byte >> 4) : (byte & 0xFu);
      const float wv = float(int(nib << 28) >> 28);
      const float wd = f16_bits_to_f32(f32_to_f16_bits(wv * f16_bits_to_f32(scale[(k / block) * N + n])));
      acc = acc + f16_bits_to_f32(a[m * K + k]) * wd;
    }
    y[e] = uint16_t(f32_to_f16_bits(acc));
  }
}

// Weight re-layout: packed [K,N] nibbles -> fragment order described at the top.
// One thread per output dword.  (w_kn_packed, wp, K, N) ; K % 64 == 0.
extern "C" __global__ void __launch_bounds__(256) mtrt_w4_prepack(const uint8_t* __restrict__ w_kn_packed,
                                                                uint32_t* __restrict__ wp, int64_t K, int64_t N) {
  const int64_t kblocks = K / BKH;
  const int64_t ntiles = (N + 31) / 32;
  const int64_t total = ntiles * kblocks * 256;
  for (int64_t d = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; d < total; d += int64_t(gridDim.x) * blockDim.x) {
    const int j = int(d & 3), lane = int((d >> 2) & 63);
    const int64_t kb = (d >> 8) % kblocks, tile = (d >> 8) / kblocks;
    const int h = lane >> 5;
    const int64_t n = tile * 32 + (lane & 31);
    const int64_t k0 = kb * BKH + 8 * (2 * j + h);
    uint32_t w = 0;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      uint32_t nib = 0;                                 // columns past N: value 0
      if (n < N) {
        const int64_t i = (k0 + q) * N + n;
        const uint32_t byte = w_kn_packed[i >> 1];
        nib = (i & 1) ? (byte >> 4) : (byte & 0xFu);
      }
      const uint32_t u = (nib ^ 8u) & 0xFu;             // value + 8
      const int pos = (q & 1) ? (q >> 1) + 4 : (q >> 1);
      w |= u << (4 * pos);
    }
    wp[d] = w;
  }
}

}  // namespace gemm_w4a16_cluster
