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
// each with its own L2.  XCD x is given the N panels x, x+8, ... and walks down all M
// tiles of a panel before the next, so a B panel is fetched into one L2 only.  The
// grid is padded to 8 * ceil(panels / 8) * tiles_m; surplus workgroups leave at once.
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
constexpr int LDS_BYTES = 2 * STAGE;                   // 128 KiB (output staging needs 4 * kOutWave + 1 KiB, less)

__device__ __forceinline__ int lds_off(int row, int chunk) { return row * BKB + ((chunk ^ ((row >> 1) & 7)) << 4); }

typedef __attribute__((address_space(3))) void lds_void_t;
typedef __attribute__((address_space(1))) const void global_void_t;

// Byte operand [rows, row_bytes] -> one 256-row LDS panel per slice, by direct-to-LDS loads.
// A panel is 32 groups of 8 rows (1 KiB each); wave w moves groups 8w .. 8w+7.  In a group
// lane l owns LDS slot l = (row l >> 3, chunk position l & 7) and therefore fetches chunk
// (l & 7) ^ swizzle(row) of that row.
struct DmaLoader {
  uint32_t off[8];
  const int8_t* base;
  __device__ __forceinline__ void init(const int8_t* operand, int64_t rows, int64_t row_bytes, int64_t r0) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    base = operand;
#pragma unroll
    for (int g = 0; g < 8; ++g) {
      const int lrow = (wave * 8 + g) * 8 + (lane >> 3);
      int64_t row = r0 + lrow;
      row = row < rows ? row : rows - 1;               // rows past the edge re-read the last row; never stored
      off[g] = uint32_t(row * row_bytes + (((lane & 7) ^ ((lrow >> 1) & 7)) << 4));
    }
  }
  __device__ __forceinline__ void issue(int64_t slice, int8_t* panel) {
    const int wave = threadIdx.x >> 6;
    const int8_t* src = base + slice * BKB;
#pragma unroll
    for (int g = 0; g < 8; ++g)
      __builtin_amdgcn_global_load_lds((global_void_t*)(src + off[g]), (lds_void_t*)(panel + (wave * 8 + g) * 1024), 16, 0, 0);
  }
  __device__ __forceinline__ void commit(int8_t*) {}
};

// all of this wave's outstanding loads and LDS accesses are done; then meet the other waves
__device__ __forceinline__ void drain_and_barrier() {
  __asm__ volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

struct Frags {
  v4i a[4];
  v4i b[4];
};

__device__ __forceinline__ void read_frags(Frags& f, const int8_t* pa, const int8_t* pb, int wm, int wn, int frow, int chunk) {
#pragma unroll
  for (int i = 0; i < 4; ++i) f.a[i] = *reinterpret_cast<const v4i*>(pa + lds_off(wm * 128 + i * 32 + frow, chunk));
#pragma unroll
  for (int j = 0; j < 4; ++j) f.b[j] = *reinterpret_cast<const v4i*>(pb + lds_off(wn * 128 + j * 32 + frow, chunk));
}

// Traits: Acc (16-wide accumulator vector), mfma(a, b, acc), zero().
// BLoader: issue(slice, lds panel) starts the fetch of a 256-row B panel, commit(lds panel)
//          finishes it (nothing for direct-to-LDS loads; dequantise + ds_write for int4).
// Epilogue: setup(lds scratch, m0, M), column(col, N), convert4(acc, q, row in tile, bits).
template <class Traits, class BLoader, class Epilogue>
__device__ __forceinline__ void run(const int8_t* __restrict__ a, int64_t a_row_bytes, BLoader& bl, Epilogue& epi,
                                    uint16_t* __restrict__ y, int64_t M, int64_t N, int64_t slices, int64_t m0,
                                    int64_t n0, int8_t* lds) {
  using Acc = typename Traits::Acc;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;             // 2 x 2 waves: 128 x 128 each
  const int frow = lane & 31, fhalf = lane >> 5;

  Acc acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = Traits::zero();

  const int64_t last = slices - 1;
  DmaLoader al;
  al.init(a, M, a_row_bytes, m0);
  Frags f0, f1;
  al.issue(0, lds);
  bl.issue(0, lds + A_BYTES);
  bl.commit(lds + A_BYTES);
  drain_and_barrier();
  read_frags(f0, lds, lds + A_BYTES, wm, wn, frow, fhalf);

  auto mfma_all = [&](const Frags& f) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = Traits::mfma(f.a[i], f.b[j], acc[i][j]);
  };

  for (int64_t s = 0; s < slices; ++s) {
    const int cur = int(s & 1);
    const int8_t* pa = lds + cur * STAGE;
    const int8_t* pb = pa + A_BYTES;
    int8_t* na = lds + (cur ^ 1) * STAGE;
    const int64_t s1 = s + 1 < last ? s + 1 : last;
    al.issue(s1, na);
    bl.issue(s1, na + A_BYTES);
    read_frags(f1, pa, pb, wm, wn, frow, 2 + fhalf);
    mfma_all(f0);
    read_frags(f0, pa, pb, wm, wn, frow, 4 + fhalf);
    mfma_all(f1);
    read_frags(f1, pa, pb, wm, wn, frow, 6 + fhalf);
    mfma_all(f0);
    bl.commit(na + A_BYTES);
    drain_and_barrier();                                 // slice s+1 is in LDS for everybody
    read_frags(f0, na, na + A_BYTES, wm, wn, frow, fhalf);
    mfma_all(f1);
  }

  __syncthreads();                                     // every wave is done with the operand stages
  epi.setup(lds + 4 * kOutWave, m0, M);
  __syncthreads();
  int8_t* out = lds + wave * kOutWave;
  const bool vec_ok = (N % 8 == 0) && ((reinterpret_cast<uintptr_t>(y) & 15) == 0);
#pragma unroll
  for (int half = 0; half < 2; ++half) {
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
      const int j = half * 2 + jj;
      const int64_t col = n0 + wn * 128 + j * 32 + frow;
      epi.column(col, N);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int lrow = i * 32 + q * 8 + fhalf * 4;   // rows lrow .. lrow+3 <-> r = 4q .. 4q+3
          uint32_t bits[4];
          epi.convert4(acc[i][j], q, wm * 128 + lrow, bits);
#pragma unroll
          for (int e = 0; e < 4; ++e)
            *reinterpret_cast<uint16_t*>(out + (lrow + e) * kOutRow + (jj * 32 + frow) * 2) = uint16_t(bits[e]);
        }
    }
    // each wave reads back only what it wrote itself: no workgroup barrier needed
#pragma unroll
    for (int it = 0; it < 16; ++it) {
      const int lrow = it * 8 + (lane >> 3), ch = lane & 7;
      const int64_t row = m0 + wm * 128 + lrow;
      const int64_t col = n0 + wn * 128 + half * 64 + ch * 8;
      const u32x4 v = *reinterpret_cast<const u32x4*>(out + lrow * kOutRow + ch * 16);
      if (row < M) {
        if (vec_ok) {
          if (col < N) *reinterpret_cast<u32x4*>(y + row * N + col) = v;
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (col + e < N) y[row * N + col + e] = uint16_t(v[e >> 1] >> (16 * (e & 1)));
        }
      }
    }
  }
}

// Workgroup id -> tile origin with the XCD-aware order described above; false = no tile.
__device__ __forceinline__ bool tile_origin(int64_t M, int64_t N, int64_t& m0, int64_t& n0) {
  const int64_t tiles_m = (M + BM - 1) / BM;
  const int64_t panels = (N + BN - 1) / BN;
  const int64_t xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
  const int64_t panel = (local / tiles_m) * 8 + xcd;
  if (panel >= panels) return false;
  m0 = (local % tiles_m) * BM;
  n0 = panel * BN;
  return true;
}

}  // namespace gemm_core
