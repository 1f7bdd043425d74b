// Shared main loop of the two MFMA GEMM clusters (W8A8 int8 and W4A16 f16).
//
// Both compute y[M,N] from an A operand that is K-contiguous per row ([M, Kbytes] bytes)
// and a B operand that ends up K-contiguous per column in LDS; an MFMA fragment is
// 16 bytes per lane for either type (16 int8 or 8 f16), so one loop serves both.
//
// Shape.  One workgroup of 4 waves computes a 256 x 256 tile, each wave a 128 x 128
// sub-tile = 4 x 4 MFMA tiles of 32 x 32 (256 accumulator registers per lane, one
// workgroup per CU, one wave per SIMD).  Measurements on the 256 x 128 predecessor
// (wave tile 4 x 2) showed the loop bound by LDS traffic, not by the matrix cores:
// per k-step a wave read 6 KiB of fragments for 8 MFMAs (0.75 KiB/MFMA), and all
// LDS reads + writes of a 128-byte K slice needed more LDS cycles than its MFMAs
// needed matrix-core cycles.  The 4 x 4 wave tile reads 8 KiB per 16 MFMAs
// (0.5 KiB/MFMA) and halves the global->LDS bytes per MFMA as well.
//
// K advances in slices of 128 bytes, so every row segment fetched from memory is a
// whole cache line (64-byte segments made the L1 fetch twice the useful bytes).  Byte
// operands go from global memory STRAIGHT INTO LDS (global_load_lds_dwordx4: no staging
// registers, no ds_write traffic); a lane's 16 bytes land at LDS base + 16*lane, so the
// XOR swizzle is applied on the source side (the lane picks which chunk of the row it
// fetches).  Two LDS stages: the loads of slice s+1 are issued before slice s is
// multiplied and must have landed before its last k-step (s_waitcnt vmcnt(0) + barrier);
// the first fragments of slice s+1 are read right after the barrier, under the last
// k-step's MFMAs.  Inside a slice the fragments of k-step t+1 are read into a second
// register set while the 16 MFMAs of k-step t issue.  The loop body has no branches
// (past the end it re-loads the last slice into the stage nobody reads).
// The compiler does not model the LDS written by those loads, so the barrier is the
// raw s_barrier framed by explicit waits and compiler memory fences instead of
// __syncthreads (whose release fence would drain every outstanding load each time).
//
// LDS rows are 128 B (8 chunks of 16 B); chunk c of row r lives at chunk position
// c ^ ((r >> 1) & 7): conflict-free for the 16-byte fragment reads of consecutive rows
// (SQ_LDS_BANK_CONFLICT reads 0 for these kernels).
//
// Tile order: the hardware deals consecutive workgroup ids round-robin to the 8 XCDs,
// each with its own L2.  Every XCD is given the same number of tiles, neighbours in an order
// that keeps a B panel's M tiles together (tile_of_even); the grid is padded to a multiple
// of 8, surplus workgroups leave at once.
//
// Epilogue: in a 32 x 32 accumulator tile lane l holds column (l & 31) and rows
// 8*(r/4) + 4*(l >> 5) + (r % 4): 16 values in 16 different rows.  Each wave parks its
// converted sub-tile (in two halves of 64 columns) in LDS, rows padded to 144 B, and
// writes it out as whole 128-byte row segments, 16 bytes per lane.
#pragma once
#include "common.hpp"

namespace gemm_core {

using namespace mtrt_dev;

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int BM = 256, BN = 256, BKB = 128;           // tile; K slice in bytes
constexpr int THREADS = 256;
constexpr int A_BYTES = BM * BKB, B_BYTES = BN * BKB, STAGE = A_BYTES + B_BYTES;
constexpr int kOutRow = 144;                           // bytes per LDS row of the output staging (64 f16 + pad)
constexpr int kOutWave = 128 * kOutRow;
constexpr int LDS_BYTES = 2 * STAGE;                   // 128 KiB (output staging of 4 waves needs 4 * kOutWave + 2 KiB, less)
constexpr int LDS_BYTES_8WAVES = 8 * kOutWave + 2048;  // 146 KiB: output staging of 8 waves (the A ring needs 128 KiB)

__device__ __forceinline__ int lds_off(int row, int chunk) { return row * BKB + ((chunk ^ ((row >> 1) & 7)) << 4); }

typedef __attribute__((address_space(3))) void lds_void_t;
typedef __attribute__((address_space(1))) const void global_void_t;

template <int V>
struct IntC {
  static constexpr int value = V;
};

// Byte operand [rows, row_bytes] -> one 256-row LDS panel per slice, by direct-to-LDS loads.
// A panel is 32 groups of 8 rows (1 KiB each); wave w moves groups 8w .. 8w+7.  In a group
// lane l owns LDS slot l = (row l >> 3, chunk position l & 7) and therefore fetches chunk
// (l & 7) ^ swizzle(row) of that row.
template <int G>                                       // G = 32 / waves: groups each wave moves
struct DmaLoaderT {
  uint32_t off[G];
  const int8_t* base;
  int wave_u;                                          // wave index as a scalar: the LDS base of a load must be uniform
  __device__ __forceinline__ void init(const int8_t* operand, int64_t rows, int64_t row_bytes, int64_t r0) {
    const int lane = threadIdx.x & 63;
    wave_u = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    base = operand;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const int lrow = (wave_u * G + g) * 8 + (lane >> 3);
      int64_t row = r0 + lrow;
      row = row < rows ? row : rows - 1;               // rows past the edge re-read the last row; never stored
      off[g] = uint32_t(row) * uint32_t(row_bytes) + uint32_t(((lane & 7) ^ ((lrow >> 1) & 7)) << 4);   // the operand is below 4 GiB
    }
  }
  // group g (of G) of this wave's share of slice `slice`
  __device__ __forceinline__ void dma(int64_t slice, int8_t* panel, int g) const {
    __builtin_amdgcn_global_load_lds((global_void_t*)(base + slice * BKB + off[g]), (lds_void_t*)(panel + (wave_u * G + g) * 1024), 16, 0, 0);
  }
  // The same from the slice's (uniform) address: scalar base + 32-bit lane offset in the instruction itself.  The
  // offset is made opaque at the load so that its widening to 64 bits is not hoisted out of the loop (the load
  // would then take a vector address pair and one 64-bit vector add per instruction).
  __device__ __forceinline__ const int8_t* slice_base(uint32_t slice) const { return base + uint64_t(slice) * BKB; }
  __device__ __forceinline__ void dma_at(const int8_t* sbase, int8_t* panel, int g) {
    __asm__ volatile("" : "+v"(off[g]));
    __builtin_amdgcn_global_load_lds((global_void_t*)(sbase + off[g]), (lds_void_t*)(panel + (wave_u * G + g) * 1024), 16, 0, 0);
  }
};
using DmaLoader = DmaLoaderT<8>;

// all of this wave's outstanding loads and LDS accesses are done; then meet the other waves
__device__ __forceinline__ void drain_and_barrier() {
  __builtin_amdgcn_s_waitcnt(0x0070);                  // vmcnt(0) lgkmcnt(0), visible to the compiler's wait-count pass
  __asm__ volatile("s_barrier" ::: "memory");
}

template <int JT>
struct Frags {
  v4i a[4];
  v4i b[JT];
};

// Accumulators -> y.  acc[i][j] holds the TRANSPOSED 32 x 32 tile (B fragment first): lane l
// <-> output row i*32 + (l & 31), register r <-> output column j*32 + 8*(r/4) + 4*(l >> 5) + (r % 4),
// so a lane owns runs of 4 consecutive outputs of a row.  Each wave parks its converted 128 x 128
// sub-tile (in two halves of 64 columns) in LDS with 8-byte stores, rows padded to 144 B, and
// writes it out as whole 128-byte row segments, 16 bytes per lane.
// SLOTS waves own a sub-tile each (slot = wm * NWN + wn, 128 rows x 32*JT columns); `active` is
// false for waves that only take part in the barriers.
// IT (deduced): 32-row tiles per wave; the staging holds 128 rows, taller waves go through it IT / 4 times.
template <int JT, int NWN, int SLOTS, int IT, class Acc, class Epilogue>
__device__ __forceinline__ void write_tile(Acc (&acc)[IT][JT], Epilogue& epi, uint16_t* __restrict__ y, int64_t M, int64_t N,
                                           int64_t m0, int64_t n0, int8_t* lds, int slot, bool active) {
  static_assert(IT % 4 == 0, "waves cover whole groups of 128 rows");
  constexpr int WCOLS = 32 * JT;
  constexpr int HC = JT >= 2 ? 2 : 1;                  // column tiles staged at a time: 64 or 32 columns
  const int lane = threadIdx.x & 63;
  const int wm = slot / NWN, wn = slot % NWN;
  const int frow = lane & 31, fhalf = lane >> 5;
  __syncthreads();                                     // every wave is done with the operand stages
  epi.setup(lds + SLOTS * kOutWave, m0, M, n0, N);
  __syncthreads();
  if (!active) return;
  int8_t* out = lds + slot * kOutWave;
  const bool vec_ok = (N % 8 == 0) && ((reinterpret_cast<uintptr_t>(y) & 15) == 0);
  // all rows of the workgroup's tile lie inside y (the rows of all SLOTS / NWN wave rows)
  const bool rows_inside = vec_ok && m0 + (SLOTS / NWN) * (32 * IT) <= M;
  // one pass: 128 rows (row group ib) x HCP column tiles starting at column tile jt0 of the wave
  auto pass = [&](auto hcp, int ib, int jt0) {
    constexpr int HCP = decltype(hcp)::value;
    constexpr int CHUNKS = HCP * 4;                    // 16-byte chunks per staged row
    const int wrow = wm * (32 * IT) + ib * 128;         // first row of this pass inside the workgroup's tile
    const int64_t pcol = n0 + wn * WCOLS + jt0 * 32;    // first column of this pass
    if (pcol >= N) return;                             // a tile that hangs over the last column: nothing to store
    const bool inside = rows_inside && pcol + 32 * HCP <= N;
    // what the epilogue needs per column (the same for every row of the pass) is fetched once, before the rows
    epi.template columns<HCP>(wn * WCOLS + jt0 * 32 + fhalf * 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int lrow = i * 32 + frow;
      epi.row(wrow + lrow);
#pragma unroll
      for (int jj = 0; jj < HCP; ++jj)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int lcol = jj * 32 + q * 8 + fhalf * 4;  // columns lcol .. lcol+3 of this group <-> r = 4q .. 4q+3
          uint32_t words[2];                             // four 16-bit outputs, the first in the low half of words[0]
          epi.convert4(acc[ib * 4 + i][jt0 + jj], q, jj, words);
          u32x2 packed;
          packed[0] = words[0];
          packed[1] = words[1];
          *reinterpret_cast<u32x2*>(out + lrow * kOutRow + lcol * 2) = packed;
        }
    }
    // each wave reads back only what it wrote itself: no workgroup barrier needed
    if (inside) {
      // every row and column of the tile exists and whole vectors can be stored: no test per store, and the address
      // moves on by a constant (the general form below costs about ten branches and a 64-bit multiply per store)
      const int r0 = lane / CHUNKS, ch = lane % CHUNKS;
      uint16_t* dst = y + (m0 + wrow + r0) * N + (n0 + wn * WCOLS + jt0 * 32 + ch * 8);
      const int64_t step = int64_t(64 / CHUNKS) * N;
#pragma unroll
      for (int it = 0; it < 128 * CHUNKS / 64; ++it) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(out + (it * (64 / CHUNKS) + r0) * kOutRow + ch * 16);
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(dst));
        dst += step;
      }
      return;
    }
#pragma unroll
    for (int it = 0; it < 128 * CHUNKS / 64; ++it) {
      const int lrow = it * (64 / CHUNKS) + lane / CHUNKS, ch = lane % CHUNKS;
      const int64_t row = m0 + wrow + lrow;
      const int64_t col = n0 + wn * WCOLS + jt0 * 32 + ch * 8;
      const u32x4 v = *reinterpret_cast<const u32x4*>(out + lrow * kOutRow + ch * 16);
      if (row < M) {
        if (vec_ok) {
          if (col < N) __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(y + row * N + col));
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (col + e < N) y[row * N + col + e] = uint16_t(v[e >> 1] >> (16 * (e & 1)));
        }
      }
    }
  };
#pragma unroll
  for (int ib = 0; ib < IT / 4; ++ib) {
#pragma unroll
    for (int half = 0; half < JT / HC; ++half) pass(IntC<HC>{}, ib, half * HC);
    if constexpr (JT % HC != 0) pass(IntC<1>{}, ib, JT - 1);   // an odd tile left over: 32 columns
  }
}

// The same sub-tiles written as f32, straight from the accumulators: a lane's runs of four consecutive outputs of a
// row are one 16-byte store each (32-byte pieces of a row per half wave, merged in the write-back cache); no staging.
// Epilogue: finish4(values of columns col .. col+3, col, N).  For the 2 x 2 waves of `run`.
template <int JT, class Acc, class Epilogue>
__device__ __forceinline__ void write_tile_f32(Acc (&acc)[4][JT], Epilogue& epi, float* __restrict__ y, int64_t M, int64_t N,
                                               int64_t m0, int64_t n0, int wave) {
  const int lane = threadIdx.x & 63;
  const int wm = wave >> 1, wn = wave & 1;
  const int frow = lane & 31, fhalf = lane >> 5;
  const bool vec_ok = (N % 4 == 0) && ((reinterpret_cast<uintptr_t>(y) & 15) == 0);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t row = m0 + wm * 128 + i * 32 + frow;
    if (row >= M) continue;
#pragma unroll
    for (int j = 0; j < JT; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int64_t col = n0 + wn * (32 * JT) + j * 32 + q * 8 + fhalf * 4;
        if (col >= N) continue;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc[i][j][4 * q + e];
        epi.finish4(v, col, N);
        if (vec_ok && col + 3 < N) {
          const f32x4 t = {v[0], v[1], v[2], v[3]};
          __builtin_nontemporal_store(t, reinterpret_cast<f32x4*>(y + row * N + col));
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (col + e < N) y[row * N + col + e] = v[e];
        }
      }
  }
}
template <int JT, class Acc, class Epilogue>
__device__ __forceinline__ void finish_tile(Acc (&acc)[4][JT], Epilogue& epi, uint16_t* __restrict__ y, int64_t M, int64_t N,
                                            int64_t m0, int64_t n0, int8_t* lds, int wave) {
  write_tile<JT, 2, 4>(acc, epi, y, M, N, m0, n0, lds, wave, true);
}
template <int JT, class Acc, class Epilogue>
__device__ __forceinline__ void finish_tile(Acc (&acc)[4][JT], Epilogue& epi, float* __restrict__ y, int64_t M, int64_t N,
                                            int64_t m0, int64_t n0, int8_t*, int wave) {
  write_tile_f32<JT>(acc, epi, y, M, N, m0, n0, wave);
}

// Both operands as bytes, K-contiguous per row / per column: a [M, a_row_bytes], b [N, a_row_bytes].
// 4 waves (2 x 2) compute a 256 x (64 * JT) tile: JT = 4 is the full tile, JT = 2 the half-width
// tile that fills the last, partial round of a launch.
// Traits: Acc (16-wide accumulator vector), mfma(first, second, acc), zero().
// Epilogue: setup(lds scratch, m0, M, n0, N), columns<HC>(first column of the lane in the tile), row(row in tile),
// convert4(acc, q, column tile of the pass, words): outputs 4q .. 4q+3 of the accumulator as two words of two.
// Y: uint16_t (16-bit outputs through the staged epilogue) or float (direct stores, see write_tile_f32).
template <class Traits, int JT, class Epilogue, typename Y>
__device__ __forceinline__ void run(const int8_t* __restrict__ a, const int8_t* __restrict__ b, int64_t row_bytes, Epilogue& epi,
                                    Y* __restrict__ y, int64_t M, int64_t N, int64_t slices, int64_t m0,
                                    int64_t n0, int8_t* lds) {
  using Acc = typename Traits::Acc;
  constexpr int GB = 2 * JT;                           // direct-to-LDS loads per wave and slice for the B panel
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;             // 2 x 2 waves: 128 x (32 * JT) each
  const int frow = lane & 31, fhalf = lane >> 5;

  Acc acc[4][JT];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < JT; ++j) acc[i][j] = Traits::zero();

  const int64_t last = slices - 1;
  DmaLoaderT<8> al;
  al.init(a, M, row_bytes, m0);
  DmaLoaderT<GB> bl;
  bl.init(b, N, row_bytes, n0);
  Frags<JT> f0, f1;

  auto read_a = [&](Frags<JT>& f, const int8_t* pa, int chunk, int i) {
    f.a[i] = *reinterpret_cast<const v4i*>(pa + lds_off(wm * 128 + i * 32 + frow, chunk));
  };
  auto read_b = [&](Frags<JT>& f, const int8_t* pb, int chunk, int j) {
    f.b[j] = *reinterpret_cast<const v4i*>(pb + lds_off(wn * (32 * JT) + j * 32 + frow, chunk));
  };
  // fragment n of a k-step in the order the MFMAs consume them: a0, b0 .. b(JT-1), a1, a2, a3
  auto read_nth = [&](Frags<JT>& f, const int8_t* pa, const int8_t* pb, int chunk, int n) {
    if (n == 0) read_a(f, pa, chunk, 0);
    else if (n <= JT) read_b(f, pb, chunk, n - 1);
    else read_a(f, pa, chunk, n - JT);
  };

#pragma unroll
  for (int g = 0; g < 8; ++g) al.dma(0, lds, g);
#pragma unroll
  for (int g = 0; g < GB; ++g) bl.dma(0, lds + A_BYTES, g);
  drain_and_barrier();
#pragma unroll
  for (int n = 0; n < 4 + JT; ++n) read_nth(f0, lds, lds + A_BYTES, fhalf, n);

  // One K slice = 4 k-steps = 4 x 8 chunks.  A chunk is JT/2 MFMAs, one fragment read for the
  // next k-step (two in chunk 0, none in the last ones, so that the wait in front of the next
  // k-step finds them done) and in k-step 0 its share of the loads of the next slice, fenced so
  // that the compiler keeps the interleave as written (left alone it gathers the LDS reads in
  // front of the MFMAs that need them and the matrix cores idle for an LDS round trip every
  // k-step).  A wave's own LDS and memory instructions take their issue cycles out of its MFMA
  // stream, so there are as few of them as the tile shape allows.
  auto kstep = [&](auto step, const Frags<JT>& cur, Frags<JT>& nxt, const int8_t* ra, const int8_t* rb, int chunk,
                   int64_t s1, int8_t* na, int8_t* nb) {
    constexpr int P = decltype(step)::value;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const int i = c >> 1, j = (c & 1) * (JT / 2);
#pragma unroll
      for (int jj = 0; jj < JT / 2; ++jj) acc[i][j + jj] = Traits::mfma(cur.b[j + jj], cur.a[i], acc[i][j + jj]);
      if (c == 0) {
        read_nth(nxt, ra, rb, chunk, 0);
        read_nth(nxt, ra, rb, chunk, 1);
      } else if (c + 1 < 4 + JT) {
        read_nth(nxt, ra, rb, chunk, c + 1);
      }
      if (P == 0) {
        al.dma(s1, na, c);
        if (c < GB) bl.dma(s1, nb, c);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto slice_body = [&](auto par, int64_t s) {
    constexpr int PAR = decltype(par)::value;
    const int8_t* pa = lds + PAR * STAGE;
    const int8_t* pb = pa + A_BYTES;
    int8_t* na = lds + (PAR ^ 1) * STAGE;
    int8_t* nb = na + A_BYTES;
    const int64_t s1 = s + 1 < last ? s + 1 : last;
    kstep(IntC<0>{}, f0, f1, pa, pb, 2 + fhalf, s1, na, nb);
    kstep(IntC<1>{}, f1, f0, pa, pb, 4 + fhalf, s1, na, nb);
    kstep(IntC<2>{}, f0, f1, pa, pb, 6 + fhalf, s1, na, nb);
    drain_and_barrier();                                 // slice s+1 is in LDS for everybody
    kstep(IntC<3>{}, f1, f0, na, nb, fhalf, s1, na, nb);
  };

  int64_t s = 0;
  for (; s + 1 < slices; s += 2) {                     // no branch inside: the loop body stays one basic block
    slice_body(IntC<0>{}, s);
    slice_body(IntC<1>{}, s + 1);
  }
  if (s < slices) slice_body(IntC<0>{}, s);

  finish_tile<JT>(acc, epi, y, M, N, m0, n0, lds, wave);
}

// Tile order.  The hardware deals consecutive workgroup ids round-robin to the 8 XCDs, each with its own L2, so
// workgroup id belongs to XCD id % 8.  All tiles are put in ONE order: M tiles in groups of `group`; inside a group the
// panels one after the other, a panel's M tiles of the group next to each other.  An XCD's 32 units then work on
// `group` M tiles x 32 / group panels at a time, and what its L2 has to fetch per K slice is group x (A panel slice)
// + 32 / group x (B panel slice): the group size that minimises it depends on the bytes per row of the two operands
// (for 4-bit weights under f16 activations a B slice is a quarter of an A slice, so few M tiles and many panels
// re-read far less; group >= tiles_m walks down all M tiles of a panel before the next).
// XCD x takes the tiles [x * per, (x + 1) * per) of that order, per = nblocks / 8 = ceil(tiles / 8): every XCD gets the
// same number of tiles, give or take one.  Dealing whole panels to the XCDs (panel p to XCD p % 8: a panel is then
// fetched into one L2 only) leaves some XCDs with a panel more than others, and on real data a launch lasts as long
// as its busiest XCD, whose clock follows its load: W4A16 M = 4096 with 43 panels, XCDs with 96 and with 80 tiles,
// 324 us; 86 each, 297 us (on zero operands the same either way).  A panel that straddles two XCDs' ranges is fetched
// into two L2s.
// nblocks = even_blocks(tiles): ids of this section of the grid (8 * per); surplus ids get no tile.
// (Tile counts fit 32 bits: the index arithmetic is 32-bit on purpose.  As 64-bit divisions, which the hardware does
// not have, it was some 500 scalar instructions, over a microsecond, in front of the first load of every workgroup.)
__device__ __host__ __forceinline__ int64_t even_blocks(int64_t tiles) { return 8 * ((tiles + 7) / 8); }
__device__ __forceinline__ bool tile_of_even(uint32_t id, uint32_t nblocks, int64_t tiles_m64, int64_t panels64, int64_t group64,
                                             int64_t& tile_m, int64_t& panel) {
  const uint32_t tiles_m = uint32_t(tiles_m64), panels = uint32_t(panels64);
  const uint32_t group = uint32_t(group64) < tiles_m ? uint32_t(group64) : tiles_m;
  const uint32_t per = nblocks >> 3;
  const uint32_t at = (id & 7) * per + (id >> 3);
  if (at >= tiles_m * panels) return false;
  const uint32_t per_group = panels * group;
  const uint32_t full = tiles_m / group;                 // whole groups; a last group holds the remainder
  uint32_t g = at / per_group, r, size;
  if (g < full) {
    r = at - g * per_group;
    size = group;
  } else {
    g = full;
    r = at - full * per_group;
    size = tiles_m - full * group;
  }
  const uint32_t q = r / size;
  panel = q;
  tile_m = g * group + (r - q * size);
  return true;
}

// ---- any row length, any alignment ----------------------------------------------------------------------
// The tile loop for operands the loop above does not take (rows that are not whole 128-byte slices, operands off
// 16-byte alignment or of 4 GiB and more).  Both operands as bytes, K-contiguous per row: a [M, row_bytes],
// b [N, row_bytes].  128 x 128 tiles, four waves (2 x 2) of 64 x 64; a k-step of 128 bytes per row goes through
// registers into one LDS stage (row pitch 144 bytes: the sixteen rows of a fragment read start in sixteen different
// groups of four banks), the next k-step's global loads in flight while the MFMAs of this one run.  Global
// accesses are 16 bytes at byte alignment; the chunk that straddles the end of a row is read byte by byte (in the last
// k-step only, so that no other step's loads wait on that loop) and padded with zeros (a zero in both operands: the padded products are exact zeros for integers and floats alike), rows
// past M / N read as zeros.  16-bit outputs are staged through the same LDS so that the stores are whole 128-byte
// row pieces; 32-bit outputs go out as 16-byte pieces straight from the accumulators.
// Traits as for `run`.  Epilogue: row(row, row < M) once per output row of the lane, then finish(sum, col, col < N)
// per element: the 16-bit pattern (Y = uint16_t) or the float (Y = float) to store.
// Grid: any; workgroup g takes tiles g, g + gridDim.x, ... (all row tiles of one 128-column panel are neighbours).
namespace edge {
constexpr int kTile = 128, kStep = 128, kPitch = 144;
constexpr int kLdsBytes = 2 * kTile * kPitch;
typedef u32x4 u32x4_bytes __attribute__((aligned(1)));
typedef u32x4 u32x4_halves __attribute__((aligned(2)));
typedef f32x4 f32x4_words __attribute__((aligned(4)));

// A 16-byte chunk that lies wholly inside its row; zeros otherwise (rows past the last one, the chunk that straddles
// the end of a row: see finish_chunk).  No loop in here: the callers' loads stay in flight together.
__device__ __forceinline__ u32x4 load_chunk(const int8_t* __restrict__ base, int64_t row, int64_t rows, int64_t row_bytes, int64_t k) {
  u32x4 v = {0u, 0u, 0u, 0u};
  if (row < rows && k + 16 <= row_bytes) v = *reinterpret_cast<const u32x4_bytes*>(base + row * row_bytes + k);
  return v;
}
// The chunk that straddles the end of its row (1 .. 15 bytes inside), byte by byte; any other chunk is returned as it
// is.  Only the last k-step of rows that are not whole chunks has such a chunk: callers test that first.
__device__ __forceinline__ u32x4 finish_chunk(u32x4 v, const int8_t* __restrict__ base, int64_t row, int64_t rows, int64_t row_bytes, int64_t k) {
  if (row >= rows || k >= row_bytes || k + 16 <= row_bytes) return v;
  const int8_t* p = base + row * row_bytes + k;
  const int left = int(row_bytes - k);
  uint64_t lo = 0, hi = 0;
#pragma unroll 1
  for (int b = 0; b < left; ++b) {
    const uint64_t byte = uint8_t(p[b]);
    if (b < 8) lo |= byte << (8 * b);
    else hi |= byte << (8 * (b - 8));
  }
  v[0] = uint32_t(lo); v[1] = uint32_t(lo >> 32); v[2] = uint32_t(hi); v[3] = uint32_t(hi >> 32);
  return v;
}
// The four chunks of one operand a lane moves per k-step: rows r0 + crow + 32 i, bytes k .. k + 15.
__device__ __forceinline__ void load_chunks(u32x4 (&r)[4], const int8_t* __restrict__ base, int64_t r0, int64_t rows, int64_t row_bytes,
                                            int64_t k, bool last_step) {
  const int crow = threadIdx.x >> 3;
#pragma unroll
  for (int i = 0; i < 4; ++i) r[i] = load_chunk(base, r0 + crow + 32 * i, rows, row_bytes, k);
  if (last_step && (row_bytes & 15)) {
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = finish_chunk(r[i], base, r0 + crow + 32 * i, rows, row_bytes, k);
  }
}

// One k-step of the four waves from the two operand stages (128 rows of kPitch bytes each, kStep bytes of k per row).
template <class Traits>
__device__ __forceinline__ void multiply_stage(typename Traits::Acc (&acc)[2][2], const int8_t* sa, const int8_t* sb) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int frow = lane & 31, fhalf = lane >> 5;
#pragma unroll
  for (int p = 0; p < kStep / 32; ++p) {
    v4i fa[2], fb[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      fa[i] = *reinterpret_cast<const v4i*>(sa + (wm * 64 + i * 32 + frow) * kPitch + p * 32 + fhalf * 16);
      fb[i] = *reinterpret_cast<const v4i*>(sb + (wn * 64 + i * 32 + frow) * kPitch + p * 32 + fhalf * 16);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = Traits::mfma(fb[j], fa[i], acc[i][j]);
  }
}

// The finished 128 x 128 tile of the four waves (acc[i][j]: rows 64 wm + 32 i, columns 64 wn + 32 j) out to y through
// the epilogue; `lds` (at least kLdsBytes) is the staging of 16-bit outputs and must no longer be read as operands
// by any wave when a wave's stores begin (the barrier below), nor written again before the caller's next barrier.
template <class Acc, class Epilogue, typename Y>
__device__ __forceinline__ void write_tile(Acc (&acc)[2][2], Epilogue& epi, Y* __restrict__ y, int64_t M, int64_t N, int64_t m0,
                                           int64_t n0, int8_t* lds) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int frow = lane & 31, fhalf = lane >> 5;
  // lane (frow, fhalf) holds row frow of each 32 x 32 block, columns 8 q + 4 fhalf + e in register 4 q + e
  if constexpr (sizeof(Y) == 2) {
    __syncthreads();                                 // all fragment reads done: the stage becomes the output staging
    int8_t* out = lds + wave * (64 * kPitch);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int64_t row = m0 + wm * 64 + i * 32 + frow;
      epi.row(row, row < M);
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int lcol = j * 32 + q * 8 + fhalf * 4;
          const int64_t col = n0 + wn * 64 + lcol;
          uint32_t bits[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) bits[e] = epi.finish(acc[i][j][4 * q + e], col + e, col + e < N);
          u32x2 packed;
          packed[0] = bits[0] | (bits[1] << 16);
          packed[1] = bits[2] | (bits[3] << 16);
          *reinterpret_cast<u32x2*>(out + (i * 32 + frow) * kPitch + lcol * 2) = packed;
        }
    }
    // a wave reads back only what it wrote, and its own LDS accesses complete in order: no workgroup barrier
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const int lrow = r * 8 + (lane >> 3), lcol = (lane & 7) * 8;
      const int64_t row = m0 + wm * 64 + lrow, col = n0 + wn * 64 + lcol;
      if (row >= M || col >= N) continue;
      const u32x4 v = *reinterpret_cast<const u32x4*>(out + lrow * kPitch + lcol * 2);
      uint16_t* dst = y + row * N + col;
      if (col + 8 <= N) {
        *reinterpret_cast<u32x4_halves*>(dst) = v;
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (col + e < N) dst[e] = uint16_t(v[e >> 1] >> (16 * (e & 1)));
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int64_t row = m0 + wm * 64 + i * 32 + frow;
      epi.row(row, row < M);
      if (row >= M) continue;
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int64_t col = n0 + wn * 64 + j * 32 + q * 8 + fhalf * 4;
          if (col >= N) continue;
          f32x4 v;
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = epi.finish(acc[i][j][4 * q + e], col + e, col + e < N);
          float* dst = y + row * N + col;
          if (col + 4 <= N) {
            *reinterpret_cast<f32x4_words*>(dst) = v;
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (col + e < N) dst[e] = v[e];
          }
        }
    }
  }
}

template <class Traits, class Epilogue, typename Y>
__device__ __forceinline__ void run(const int8_t* __restrict__ a, const int8_t* __restrict__ b, int64_t row_bytes, Epilogue& epi,
                                    Y* __restrict__ y, int64_t M, int64_t N, int8_t* lds) {
  using Acc = typename Traits::Acc;
  int8_t* sa = lds;
  int8_t* sb = lds + kTile * kPitch;
  const int64_t tiles_m = (M + kTile - 1) / kTile, tiles_n = (N + kTile - 1) / kTile;
  const int64_t steps = (row_bytes + kStep - 1) / kStep;
  // the four chunks of each operand this lane moves per k-step: rows crow + 32 i, bytes ccol .. ccol + 15
  const int crow = threadIdx.x >> 3, ccol = (threadIdx.x & 7) * 16;
  for (int64_t tile = blockIdx.x; tile < tiles_m * tiles_n; tile += gridDim.x) {
    const int64_t m0 = (tile % tiles_m) * kTile, n0 = (tile / tiles_m) * kTile;
    Acc acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = Traits::zero();
    u32x4 ra[4], rb[4];
    load_chunks(ra, a, m0, M, row_bytes, ccol, steps == 1);
    load_chunks(rb, b, n0, N, row_bytes, ccol, steps == 1);
    for (int64_t s = 0; s < steps; ++s) {
      __syncthreads();                                 // the previous k-step's (or tile's) LDS reads are done
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        *reinterpret_cast<u32x4*>(sa + (crow + 32 * i) * kPitch + ccol) = ra[i];
        *reinterpret_cast<u32x4*>(sb + (crow + 32 * i) * kPitch + ccol) = rb[i];
      }
      __syncthreads();
      if (s + 1 < steps) {
        load_chunks(ra, a, m0, M, row_bytes, (s + 1) * kStep + ccol, s + 2 == steps);
        load_chunks(rb, b, n0, N, row_bytes, (s + 1) * kStep + ccol, s + 2 == steps);
      }
      multiply_stage<Traits>(acc, sa, sb);
    }
    write_tile(acc, epi, y, M, N, m0, n0, lds);
  }
}
}  // namespace edge

// ---- up to 32 rows against K-contiguous weights -----------------------------------------------------------
// a [M <= 32 MT, row_bytes], w [N, row_bytes], both in whole 128-byte slices and 16-byte aligned.  With so few rows a
// call is bound by reading the weights once, and a tile of the loops above would spend a whole K loop on padding.
// One workgroup per 32 weight rows (output columns); its WAVES waves split K.  Each wave works alone, without
// workgroup barriers: per 128-byte slice it reads its 32 weight rows and the 32 activation rows as whole rows (eight
// lanes per row, so every instruction moves 128 contiguous bytes of eight rows), parks them in two stages of its own
// in LDS (row pitch 144 bytes: conflict-free fragment reads) and multiplies the four k-steps from there; the loads of
// the next two slices are in flight meanwhile (two register sets, no branch around a load, so the waits are counted
// exactly), and the other waves of the compute unit cover the rest of the latency.  Rows past M and weight rows
// past N repeat the last valid row: they only reach outputs that are never stored.  The waves' partial sums meet in
// LDS, in wave order, and go out through the epilogue.
// Traits as for `run`, plus Scalar (the accumulator's element type).  Epilogue: finish(sum, row, col) -> the 16-bit
// pattern (Y = uint16_t) or the float (Y = float) of y[row, col].  Grid: any (tiles dealt round-robin), block = 64 WAVES.
namespace rows32 {
constexpr int kPitch = 144, kStageBytes = 32 * kPitch;
// MT: activation row tiles of 32 (1: M <= 32, 2: M <= 64, the weight fragments of a k-step serving both)
template <int WAVES, int MT = 1, bool FRAG = false> constexpr int lds_bytes() { return WAVES * (MT + (FRAG ? 0 : 1)) * kStageBytes; }

// FRAG: `w` is not the [N,K] array but its fragment-order re-layout (per 32 rows and 128-byte slice four 1 KiB blocks,
// lane l of block q holding the 16 bytes of k-step q of its row: exactly the second MFMA operand).  The weight
// fragments then go from memory to registers and into the MFMA without passing LDS, 1 KiB contiguous per instruction.
template <class Traits, int WAVES, int MT = 1, bool FRAG = false, class Epilogue, typename Y>
__device__ __forceinline__ void run(const int8_t* __restrict__ a, const int8_t* __restrict__ w, int64_t row_bytes, Epilogue& epi,
                                    Y* __restrict__ y, int64_t M, int64_t N, int8_t* lds) {
  using Acc = typename Traits::Acc;
  using Scalar = typename Traits::Scalar;
  constexpr int kWaveBytes = (MT + (FRAG ? 0 : 1)) * kStageBytes;   // fragment-order weights need no stage
  static_assert(kWaveBytes >= MT * 16 * 64 * int(sizeof(Scalar)), "a wave's stages also hold its partial sums");
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int frow = lane & 31, fhalf = lane >> 5;
  const int lrow = lane >> 3, lchunk = (lane & 7) * 16;
  const int64_t slices = row_bytes / 128;
  const int64_t kb0 = slices * wave / WAVES, kb1 = slices * (wave + 1) / WAVES;
  int8_t* sa = lds + wave * kWaveBytes;
  int8_t* sw = sa + MT * kStageBytes;
  const int64_t tiles = (N + 31) / 32;
  for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    const int8_t* ap[4 * MT];
    const int8_t* wp[4];
#pragma unroll
    for (int i = 0; i < 4 * MT; ++i) {
      const int64_t m = lrow + 8 * i;
      ap[i] = a + (m < M ? m : M - 1) * row_bytes + lchunk;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int64_t n = tile * 32 + lrow + 8 * i;
      // fragment order: block i of a slice (the re-layout holds zeros for rows past N); else: row n of the array
      wp[i] = FRAG ? w + tile * slices * 4096 + i * 1024 + lane * 16 : w + (n < N ? n : N - 1) * row_bytes + lchunk;
    }
    constexpr int64_t kSliceBytes = FRAG ? 4096 : 128;   // from one slice of a lane's weight pieces to the next
    Acc acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = Traits::zero();
    u32x4 ra[2][4 * MT], rw[2][4];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      // a slice past the wave's last one is the last one again (slice 0 for a wave without slices; slices >= 1)
      int64_t kb = kb0 + p < kb1 ? kb0 + p : kb1 - 1;
      kb = kb < 0 ? 0 : kb;
#pragma unroll
      for (int i = 0; i < 4 * MT; ++i) ra[p][i] = *reinterpret_cast<const u32x4*>(ap[i] + kb * 128);
#pragma unroll
      for (int i = 0; i < 4; ++i) rw[p][i] = *reinterpret_cast<const u32x4*>(wp[i] + kb * kSliceBytes);
    }
    for (int64_t kb = kb0; kb < kb1; kb += 2) {
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        if (kb + p < kb1) {
#pragma unroll
          for (int i = 0; i < 4 * MT; ++i) *reinterpret_cast<u32x4*>(sa + (lrow + 8 * i) * kPitch + lchunk) = ra[p][i];
          u32x4 held[4];                               // fragment order: this slice's fragments stay in registers
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            if (FRAG) held[i] = rw[p][i];
            else *reinterpret_cast<u32x4*>(sw + (lrow + 8 * i) * kPitch + lchunk) = rw[p][i];
          }
          const int64_t next = kb + p + 2 < kb1 ? kb + p + 2 : kb1 - 1;   // always a load: the waits stay countable
#pragma unroll
          for (int i = 0; i < 4 * MT; ++i) ra[p][i] = *reinterpret_cast<const u32x4*>(ap[i] + next * 128);
#pragma unroll
          for (int i = 0; i < 4; ++i) rw[p][i] = *reinterpret_cast<const u32x4*>(wp[i] + next * kSliceBytes);
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            v4i fw;
            if (FRAG) {
              fw = v4i{int(held[q][0]), int(held[q][1]), int(held[q][2]), int(held[q][3])};
            } else {
              fw = *reinterpret_cast<const v4i*>(sw + frow * kPitch + q * 32 + fhalf * 16);
            }
#pragma unroll
            for (int t = 0; t < MT; ++t) {
              const v4i fa = *reinterpret_cast<const v4i*>(sa + (t * 32 + frow) * kPitch + q * 32 + fhalf * 16);
              acc[t] = Traits::mfma(fa, fw, acc[t]);
            }
          }
        }
      }
    }
    // lane (n = lane % 32, h = lane / 32) holds rows 32 t + 8 (r / 4) + 4 h + r % 4 of column n in register r of acc[t]
    Scalar* mine = reinterpret_cast<Scalar*>(sa);
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) mine[(t * 16 + r) * 64 + lane] = acc[t][r];
    __syncthreads();
    for (int e = threadIdx.x; e < MT * 16 * 64; e += 64 * WAVES) {
      const int t = e >> 10, r = (e >> 6) & 15, l = e & 63;
      Scalar v = reinterpret_cast<const Scalar*>(lds)[e];
#pragma unroll
      for (int k = 1; k < WAVES; ++k) v = v + reinterpret_cast<const Scalar*>(lds + k * kWaveBytes)[e];
      const int64_t row = t * 32 + (r >> 2) * 8 + (l >> 5) * 4 + (r & 3);
      const int64_t c = tile * 32 + (l & 31);
      if (row < M && c < N) y[row * N + c] = Y(epi.finish(v, row, c));
    }
    __syncthreads();                                   // the sums are read before the next tile's slices land in the stages
  }
}
}  // namespace rows32

}  // namespace gemm_core
