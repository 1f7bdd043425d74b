// Part 2 of the C ABI: one entry point per kernel cluster.  Each validates its
// operands on the host (so that no launch can address memory outside them), picks
// the kernel variant and launch shape for gfx950, builds the argument array in the
// reference's kernelParams convention and launches from the built-in module.
// This is the hand-written counterpart of the get-function + launch pairs the
// reference compiler emits for its generated kernels
// (mlir-tensorrt/compiler/lib/Passes/1_Core/KernelToCUDA/KernelToCUDA.cpp:151-186;
//  mlir-tensorrt/compiler/lib/Passes/2_Host/HostToExecutor/CUDAToExecutor/CUDAToExecutor.cpp:355-413).
#include "runtime_internal.hpp"

#include <algorithm>
#include <atomic>
#include <cstdlib>

using namespace mtrt_rt;

namespace {

constexpr int kTile = 16;           // elements per lane per trip in qdq.hip
constexpr uint32_t kBlock = 256;
constexpr uint32_t kMaxGrid = 1u << 20;
// The one-wave-per-row kernels (layernorm / softmax `_v*`) map rows to waves from the workgroup index and do
// not loop, so their grid must cover every row: ceil(rows / 4) workgroups, which blocks_for() caps at
// kMaxGrid.  Tensors with more rows take the `_any` kernels, which loop over rows.
constexpr int64_t kMaxRowsPerWaveKernels = int64_t(kMaxGrid) * (kBlock / 64);

// ---- launch-time estimates behind the GEMM dispatch ------------------------------------------------------------
// Every choice between two GEMM kernels compares two estimates of the launch time in microseconds.  All constants
// live here, each with the measurement that set it (one MI355X, 256 compute units, times from HIP events over
// rotating operands; `rounds` = ceil(tiles / compute units), `row bytes` = K * element size).  They are fits to a
// few points, good to about 10 %: near a crossover either kernel is within that of the other, so a box whose power
// state moves the times by a few per cent picks differently without losing more than that.
namespace tuning {
// Tile loop against [N,K] operands (both panels through LDS), per round of 256 x 256 tiles: a fixed part plus the
// K loop.  int8: M = 16, K = 4096, N = 11008 32.7 us; M = 1, K = N = 4096 27.6 us; M = 32, K = N = 8192 57.1 us
// (8 + 0.006 * 4096 = 32.6, 8 + 0.006 * 8192 = 57.2).
constexpr double kTileFixedUs = 8.0, kTileUsPerRowByte = 0.006;
// Tile loop on fragment-order int8 weights (weights straight into registers), per round: M = 64 at (K, N) =
// (4096, 4096) 21.0 us, (4096, 11008) 23.2 us, (8192, 8192) 38.4 us; never below streaming the weights at 4.5 TB/s
// ((11008, 4096) 34.1 us for 45 MB + the fixed part).
constexpr double kFragTileFixedUs = 5.0, kFragTileUsPerK = 0.004, kFragTileBytesPerUs = 4.5e6;
// Wave-private kernels that read the weights once (gemm_core::rows32), up to 64 rows: a fixed part plus the weight
// bytes at the rate the kernel streams them.  [N,K] int8 weights 3.4 TB/s (M = 16, K = 4096, N = 11008 13.0 us;
// M = 32, K = N = 8192 18.2 us); f16 / bf16 / f32 [N,K] weights and fragment-order int8 weights 4.0 TB/s
// (dense f16 M = 16, K = 4096, N = 11008 23.4 us; fragment order M = 64 (4096, 4096) 9.3 us, (11008, 4096) 17.1 us).
constexpr double kRowsFixedUs = 3.0, kRowsBytesPerUs = 3.4e6, kRowsWideBytesPerUs = 4.0e6, kFragRowsFixedUs = 5.0;
// The same kernels with four row tiles (65 to 128 rows): one workgroup per compute unit at a time, so rounds of 32-column
// tiles, each the length of its K loop.  [N,K] operands 3.7 ns per row byte (int8 M = 128, K = N = 4096 18.4 us,
// K = N = 8192 30.7 us); fragment-order weights 3.2 ns per k (16.1 us / 28.1 us at the same shapes).
constexpr double kRows128FixedUs = 3.0, kRows128UsPerRowByte = 0.0037, kFragRows128UsPerK = 0.0032;
// W4A16 tile choice: a full round of 256 x 256 tiles takes 3.25 times a full round of 128 x 128 tiles (for four times
// the work), and a last round filled to a fraction f of the units takes 0.56 + 0.44 f^2 of a full one (fewer units
// share the power budget).  Fitted over M = 48 ... 4096 at (K, N) = (4096, 4096), (4096, 11008), (11008, 4096),
// (8192, 8192), (5120, 13824), (4096, 14336), (8192, 28672), (4096, 2048), 16 to 256 tiles in the last round; where
// the rule changed the choice: K = N = 4096, M = 2048 83.6 -> 77.1 us; N = 11008, M = 1536 193.2 -> 175.0 us.
constexpr double kW4BigRoundPerSmallRound = 3.25, kW4PartialRoundBase = 0.56, kW4PartialRoundSlope = 0.44;
// ... and a round of 256 x 384 tiles takes 1.5 x 0.95 of a round of 256 x 256 tiles (K = 4096, N = 11008, the benchmark's
// data, old and new in one process: M = 4096, 3 rounds against 2, 298.4 -> 286.8 us; M = 8192 600 -> 571; M = 2048, two
// rounds against one, 181 -> 145).
constexpr double kW4WideRoundPerBigRound = 1.5 * 0.95;
// ... and a round of 128 x 256 tiles 1.9 rounds of 128 x 128 tiles (0.48 against 0.37 us per 64-k slice and a longer
// start and end; at 15 shapes with M = 300 ... 2048, (K, N) = (4096, 11008), (4096, 4096), (11008, 4096), (8192, 8192),
// (5120, 13824) the estimate takes the fastest of the four tiles at every one).
constexpr double kW4Mid256RoundPerSmallRound = 1.9;
// W8A8 on fragment-order weights: a round of 256 x 384 tiles, in rounds of 256 x 256 tiles.  One and a half times the
// MFMAs at 0.9 of the time per MFMA (K = 4096, N = 11008, the benchmark's data, both kernels in one process: M = 2048,
// one round against one and a half, 77.9 against 83.5 us; M = 4096, two against three, 158 / 165; M = 8192, four
// against five and a half, 321 / 338; M = 3072, two against two and a half, 137 / 135).
constexpr double kW8WideRoundPerRound = 1.5 * 0.9;
} // namespace tuning

const char *float_name(int32_t dt) {
  switch (dt) {
  case MTRT_F32: return "f32";
  case MTRT_F16: return "f16";
  case MTRT_BF16: return "bf16";
  }
  return nullptr;
}
const char *code_name(int32_t dt) {
  switch (dt) {
  case MTRT_I8: return "i8";
  case MTRT_F8E4M3FN: return "f8";
  case MTRT_I4: return "i4";
  case MTRT_I4_PACKED: return "i4p";
  case MTRT_F4_PACKED: return "f4p";
  }
  return nullptr;
}
int float_bytes(int32_t dt) { return dt == MTRT_F32 ? 4 : 2; }

bool aligned(const void *p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// Element count of a [d0, d1] operand without signed overflow: false when the product does not fit in 63 bits.
bool element_count(int64_t d0, int64_t d1, int64_t *n) { return !__builtin_mul_overflow(d0, d1, n); }
// Matrix extents of the GEMM entry points: below 2^31 each, so that every product of two of them (and twice that)
// fits in 63 bits.
constexpr int64_t kMaxMatrixExtent = (int64_t(1) << 31) - 1;

uint32_t blocks_for(int64_t units, uint32_t per_block) {
  const int64_t b = (units + per_block - 1) / per_block;
  return uint32_t(std::max<int64_t>(1, std::min<int64_t>(b, kMaxGrid)));
}

// mode: 0 quantize, 1 dequantize, 2 fused
int32_t qdq_dispatch(int mode, hipStream_t stream, const void *x, int32_t x_dtype, void *q,
                     int32_t q_dtype, void *y, const float *scale, int32_t kind, int64_t d0,
                     int64_t d1, int64_t nb, int32_t flags) {
  clear_error();
  const char *xn = float_name(x_dtype);
  const char *qn = code_name(q_dtype);
  if (!xn)
    return set_error(MTRT_INVALID_ARGUMENT, "float operand dtype %d is not one of f32/f16/bf16", x_dtype);
  if (!qn)
    return set_error(MTRT_INVALID_ARGUMENT, "quantized dtype %d is not one of i8/f8E4M3FN/i4/i4-packed", q_dtype);
  if (d0 < 0 || d1 < 0)
    return set_error(MTRT_INVALID_ARGUMENT, "negative extent [%lld, %lld]", (long long)d0, (long long)d1);
  if (kind < MTRT_SCALE_UNIFORM || kind > MTRT_SCALE_COL)
    return set_error(MTRT_INVALID_ARGUMENT, "unknown scale kind %d", kind);
  if (kind != MTRT_SCALE_UNIFORM && nb <= 0)
    return set_error(MTRT_INVALID_ARGUMENT, "scale kind %d needs a positive scale count / block size, got %lld",
                     kind, (long long)nb);
  if (kind == MTRT_SCALE_COL && d0 % nb != 0)
    return set_error(MTRT_INVALID_ARGUMENT, "block size %lld does not divide the blocked extent %lld",
                     (long long)nb, (long long)d0);
  if (flags & ~(MTRT_Q_ROUND_TO_INT | MTRT_F8_REFHOST | MTRT_F8_VIA_F16))
    return set_error(MTRT_INVALID_ARGUMENT, "unknown flag bits 0x%x", flags);
  if ((flags & MTRT_F8_REFHOST) && (flags & MTRT_F8_VIA_F16))
    return set_error(MTRT_INVALID_ARGUMENT, "MTRT_F8_REFHOST and MTRT_F8_VIA_F16 name two different conversions; pass one");
  int64_t n;
  if (!element_count(d0, d1, &n) || n >= (int64_t(1) << 35))
    return set_error(MTRT_INVALID_ARGUMENT, "[%lld, %lld] elements exceed the supported 2^35", (long long)d0, (long long)d1);
  if (n == 0)
    return MTRT_OK;
  if (!scale || !q || (mode != 1 && !x) || (mode != 0 && !y))
    return set_error(MTRT_INVALID_ARGUMENT, "null operand");
  if (!aligned(mode == 1 ? y : x, float_bytes(x_dtype)) || (mode == 2 && !aligned(y, float_bytes(x_dtype))))
    return set_error(MTRT_INVALID_ARGUMENT, "float operand is not aligned to its element size");
  if (d1 == 0)
    return MTRT_OK;
  if (kind == MTRT_SCALE_UNIFORM)
    nb = 1;

  DeviceState *st = device_state();
  if (!st)
    return MTRT_RUNTIME_ERROR;

  // The group kernels move one 128-bit vector of the float operand (G elements)
  // per lane per instruction: they need that operand 128-bit aligned, the codes
  // aligned to the G codes a lane moves at once, and - whenever the scale changes
  // along or across rows - rows that are whole groups.
  const int group = x_dtype == MTRT_F32 ? 4 : 8;
  const bool nibbles = q_dtype == MTRT_I4_PACKED || q_dtype == MTRT_F4_PACKED;
  const uintptr_t q_align = nibbles ? group / 2 : group;
  bool tiles = aligned(q, q_align) && (mode == 1 || aligned(x, 16)) && (mode == 0 || aligned(y, 16));
  // The row- and column-scaled group kernels keep group, row and scale-block indices in 32 bits; a tensor
  // beyond that (64 GiB of f32 and more) takes the element-wise kernel, which indexes in 64 bits throughout.
  if (kind != MTRT_SCALE_UNIFORM)
    tiles = tiles && (d1 % group == 0) && n / group < (int64_t(1) << 32) && nb < (int64_t(1) << 32);
  if (kind == MTRT_SCALE_COL)
    tiles = tiles && aligned(scale, 16);

  // Row or column scales on rows that are not whole groups, or on operands not aligned for group accesses: a wave
  // per 64 groups of one row with accesses at element alignment (codes one per byte only: a packed byte can
  // straddle rows).  Everything else that is not `tiles`: one element per lane.
  // A per-tensor scale on unaligned operands is the row kind on one row of n elements.
  const bool ragged = !tiles && !nibbles;
  if (ragged && kind == MTRT_SCALE_UNIFORM) {
    kind = MTRT_SCALE_ROW;
    d0 = 1;
    d1 = n;
  }
  static const char *kModeName[] = {"q", "dq", "qdq"};
  static const char *kKindName[] = {"uniform", "row", "col"};
  static const char *kRaggedName[] = {"", "rowu", "colu"};
  KernelName name("mtrt_");
  name + kModeName[mode] + "_" + (tiles ? kKindName[kind] : (ragged ? kRaggedName[kind] : "any")) + "_" + xn + "_" + qn;

  int64_t n_arg = n, d1_arg = d1, nb_arg = nb;
  int32_t kind_arg = kind, flags_arg = flags;
  const void *x_arg = x;
  void *q_arg = q, *y_arg = y;
  const float *s_arg = scale;
  void *args[11];
  int na = 0;
  if (mode != 1) args[na++] = &x_arg;
  args[na++] = &q_arg;
  if (mode != 0) args[na++] = &y_arg;
  args[na++] = &s_arg;
  args[na++] = &n_arg;
  args[na++] = &d1_arg;
  args[na++] = &nb_arg;
  if (ragged) {                                        // row pitches of the float operand(s) and of the codes: contiguous here
    args[na++] = &d1_arg;
    args[na++] = &d1_arg;
  }
  if (!tiles && !ragged) args[na++] = &kind_arg;
  if (mode != 1) args[na++] = &flags_arg;

  if (tiles && kind == MTRT_SCALE_COL) {
    // one wave per (scale block, chunk of 32 rows of it, strip of 64 groups of columns): see qdq_col_strips
    const int64_t items = (d0 / nb) * ((nb + 31) / 32) * ((d1 / group + 63) / 64);
    return launch(st, name, blocks_for(items, kBlock / 64), kBlock, stream, args);
  }
  if (ragged) {
    const int64_t chunks = std::max<int64_t>(1, (d1 / group + 63) / 64);
    return launch(st, name, blocks_for(d0 * chunks, kBlock / 64), kBlock, stream, args);
  }
  const int64_t units = tiles ? (n + kTile - 1) / kTile : (nibbles ? (n + 1) / 2 : n);
  return launch(st, name, blocks_for(units, kBlock), kBlock, stream, args);
}

int32_t pick_nv(int64_t nvec_per_row) {
  for (int nv : {1, 2, 4, 8, 16})
    if (nvec_per_row <= int64_t(64) * nv)
      return nv;
  return 0;
}

// Some element-aligned (`_u`) kernels on f32 rows with eight vectors per lane come out of the compiler badly: the
// LayerNorm ones with 230 registers per lane (one wave per SIMD: f32 [4096, 8190] took 114 us against softmax's 45),
// the 1024-lane ones of both families with 1.4 KB of scratch memory per lane (whose allocation costs a launch some
// 10 us).  Their 16-vector forms take under 130 registers and no scratch, so those rows use them (a lane past the
// end of the row holds nothing).
int unaligned_nv(int32_t dtype, int nv, int lanes, bool layernorm) {
  return dtype == MTRT_F32 && nv == 8 && (layernorm || lanes == 1024) ? 16 : nv;
}

// Rows too long for one wave: a workgroup of 256 or 1024 lanes with 8 or 16 vectors per lane owns the row.
// Returns false when the row is longer than 1024 * 16 vectors.
bool pick_group(int64_t nvec_per_row, int *threads, int *nv) {
  for (int t : {256, 1024})
    for (int v : {8, 16})
      if (nvec_per_row <= int64_t(t) * v) {
        *threads = t;
        *nv = v;
        return true;
      }
  return false;
}

} // namespace

extern "C" {

int32_t mtrt_hip_amax(mtrt_stream_t stream, const void *x, int32_t dtype, int64_t n, float qmax,
                      float *amax_out, float *scale_out) {
  clear_error();
  const char *xn = float_name(dtype);
  if (!xn)
    return set_error(MTRT_INVALID_ARGUMENT, "amax input dtype %d is not one of f32/f16/bf16", dtype);
  if (n < 0)
    return set_error(MTRT_INVALID_ARGUMENT, "negative element count %lld", (long long)n);
  if (n > 0 && !x)
    return set_error(MTRT_INVALID_ARGUMENT, "null input");
  if (!aligned(x, float_bytes(dtype)))
    return set_error(MTRT_INVALID_ARGUMENT, "input is not aligned to its element size");
  DeviceState *st = device_state();
  if (!st)
    return MTRT_RUNTIME_ERROR;
  uint32_t *slot = reduction_slot(st, as_hip(stream));
  if (!slot)
    return MTRT_RUNTIME_ERROR;
  // Two workgroups per CU (8 waves), each lane keeping four 128-bit loads in flight; fewer when the
  // tensor is small.  Measured on bf16 [16384, 8192]: 1 / 2 / 3 / 4 / 8 / 16 workgroups per CU take
  // 51.3 / 40.7 / 41.8 / 41.9 / 45.7 / 48.2 us (fewer, longer contiguous streams and fewer arrivals at
  // the reduction tree); eight loads in flight per lane were 1 us slower.
  const int per_vec = dtype == MTRT_F32 ? 4 : 8;
  const int64_t nvec = n / per_vec;
  const uint32_t grid = uint32_t(std::max<int64_t>(
      1, std::min<int64_t>((nvec + int64_t(kBlock) * 4 - 1) / (int64_t(kBlock) * 4), int64_t(num_compute_units(st)) * 2)));
  const void *x_arg = x;
  int64_t n_arg = n;
  float qmax_arg = qmax;
  void *args[] = {&x_arg, &n_arg, &qmax_arg, &amax_out, &scale_out, &slot};
  return launch(st, KernelName("mtrt_amax_") + xn, grid, kBlock, as_hip(stream), args);
}

int32_t mtrt_hip_amax_scales(mtrt_stream_t stream, const void *x, int32_t dtype, int32_t scale_kind, int64_t d0, int64_t d1,
                             int64_t nb, float qmax, float *amax_out, float *scale_out) {
  clear_error();
  const char *xn = float_name(dtype);
  if (!xn)
    return set_error(MTRT_INVALID_ARGUMENT, "amax input dtype %d is not one of f32/f16/bf16", dtype);
  if (d0 < 0 || d1 < 0)
    return set_error(MTRT_INVALID_ARGUMENT, "negative extent [%lld, %lld]", (long long)d0, (long long)d1);
  if (scale_kind < MTRT_SCALE_UNIFORM || scale_kind > MTRT_SCALE_COL)
    return set_error(MTRT_INVALID_ARGUMENT, "unknown scale kind %d", scale_kind);
  int64_t n;
  if (!element_count(d0, d1, &n))
    return set_error(MTRT_INVALID_ARGUMENT, "[%lld, %lld] elements do not fit a 64-bit count", (long long)d0, (long long)d1);
  if (scale_kind == MTRT_SCALE_UNIFORM)
    return mtrt_hip_amax(stream, x, dtype, n, qmax, amax_out, scale_out);
  if (nb <= 0)
    return set_error(MTRT_INVALID_ARGUMENT, "scale kind %d needs a positive scale count / block size, got %lld", scale_kind,
                     (long long)nb);
  if (scale_kind == MTRT_SCALE_ROW && nb > d0 && d0 > 0)
    return set_error(MTRT_INVALID_ARGUMENT, "%lld scales for %lld rows", (long long)nb, (long long)d0);
  if (scale_kind == MTRT_SCALE_COL && d0 % nb != 0)
    return set_error(MTRT_INVALID_ARGUMENT, "block size %lld does not divide the blocked extent %lld", (long long)nb,
                     (long long)d0);
  if (d0 == 0 || d1 == 0)
    return MTRT_OK;                                    // no scale element has an input
  if (!x || (!amax_out && !scale_out))
    return set_error(MTRT_INVALID_ARGUMENT, "null operand");
  if (!aligned(x, float_bytes(dtype)))
    return set_error(MTRT_INVALID_ARGUMENT, "input is not aligned to its element size");
  DeviceState *st = device_state();
  if (!st)
    return MTRT_RUNTIME_ERROR;
  const int group = dtype == MTRT_F32 ? 4 : 8;
  const bool vec = d1 % group == 0 && aligned(x, 16);
  void *args[] = {&x, &d0, &d1, &nb, &qmax, &amax_out, &scale_out};
  if (scale_kind == MTRT_SCALE_ROW && vec && nb < 4 * int64_t(num_compute_units(st)) && nb <= d0) {
    // Few scales (one wave each would leave most of the chip idle): the tiles of a scale's rows (1024 vectors each)
    // are shared by several workgroups that meet in the output word by atomic max, about two workgroups per compute
    // unit in all; then the finishing launch.  Measured on f16 [65536, 1024]: nb = 64 945.6 us, nb = 8 7684 us as one
    // wave per scale; [8, 8M] with nb = 8 2387 us.
    const int64_t units = num_compute_units(st), nvec = d1 / group;
    const int64_t tiles = ((d0 + nb - 1) / nb) * ((nvec + 1023) / 1024);     // of the scale with the most rows
    const int64_t parts = std::max<int64_t>(1, std::min<int64_t>((2 * units + nb - 1) / nb, (tiles + 3) / 4));
    if (parts > 1) {
      int64_t count = nb;
      uint32_t *stage = reinterpret_cast<uint32_t *>(amax_out ? amax_out : scale_out);
      uint8_t *stage_bytes = reinterpret_cast<uint8_t *>(stage);
      uint32_t zero = 0;
      int32_t width = 4;
      void *fill_args[] = {&stage_bytes, &count, &zero, &width};
      int32_t rc = launch(st, KernelName("mtrt_fill"), blocks_for(count, kBlock), kBlock, as_hip(stream), fill_args);
      if (rc != MTRT_OK)
        return rc;
      int64_t parts_arg = parts;
      void *split_args[] = {&x, &d0, &d1, &nb, &parts_arg, &stage};
      rc = launch(st, KernelName("mtrt_amax_rows_split_") + xn, uint32_t(nb * parts), kBlock, as_hip(stream), split_args);
      if (rc != MTRT_OK)
        return rc;
      void *finish_args[] = {&stage, &count, &qmax, &amax_out, &scale_out};
      return launch(st, KernelName("mtrt_amax_finish_") + xn, blocks_for(count, kBlock), kBlock, as_hip(stream), finish_args);
    }
  }
  if (scale_kind == MTRT_SCALE_ROW) {
    const int64_t blocks = (nb + 3) / 4;
    if (blocks > int64_t(kMaxGrid) * 1024)
      return set_error(MTRT_INVALID_ARGUMENT, "%lld scales are too many for one launch", (long long)nb);
    return launch(st, KernelName(vec ? "mtrt_amax_rows_" : "mtrt_amax_rows_any_") + xn, uint32_t(blocks), kBlock,
                  as_hip(stream), args);
  }
  // A row length that is not whole vectors, or an unaligned operand: one lane per (block, column) while that gives
  // every compute unit a thousand lanes (f16 [8192, 8190], blocks of 128 rows: 44.7 us against 51.1 us for the
  // vector form at element alignment); with fewer, longer blocks the `_u` kernels, which move whole vectors at
  // element alignment, count a last partial vector and can share a block's rows (one block of 8192 rows: 2085 us
  // as one lane per column, 112.6 us shared).
  if (vec || (d0 / nb) * d1 < int64_t(num_compute_units(st)) * 1024) {
    const char *u = vec ? "" : "u_";
    const int64_t blocks = (d0 / nb) * (((d1 + group - 1) / group + 63) / 64), units = num_compute_units(st);
    if (blocks < 2 * units && nb >= 128 && (d0 / nb) * d1 < (int64_t(1) << 31)) {
      // Few, long blocks (one per-channel scale per column of a [K, N] weight): too few workgroups to pull the
      // tensor through.  Each block's rows are dealt to several workgroups (at least 32 rows each, about two
      // workgroups per compute unit in all, at most 16 per block: the atomics on one line are served one after
      // the other) that meet in the output itself, zeroed first, by atomic max on bit patterns; a last small
      // launch turns the patterns into amax and scale.  Measured on [4096, 11008], nb = 4096: f16 157.6 us as 22
      // workgroups, 24.3 / 26.3 / 32.3 / 40.8 us with 12 / 24 / 47 / 70 parts; f32 148.7 us, 37.5 / 36.8 / 36.3 us
      // with 6 / 12 / 24 parts.
      const int64_t want = std::min<int64_t>({(2 * units + blocks - 1) / blocks, nb / 32, int64_t(16)});
      const int64_t rows_per_part = (((nb + want - 1) / want) + 3) / 4 * 4, parts = (nb + rows_per_part - 1) / rows_per_part;
      int64_t count = (d0 / nb) * d1;
      uint32_t *stage = reinterpret_cast<uint32_t *>(amax_out ? amax_out : scale_out);
      uint8_t *stage_bytes = reinterpret_cast<uint8_t *>(stage);
      uint32_t zero = 0;
      int32_t width = 4;
      void *fill_args[] = {&stage_bytes, &count, &zero, &width};
      int32_t rc = launch(st, KernelName("mtrt_fill"), blocks_for(count, kBlock), kBlock, as_hip(stream), fill_args);
      if (rc != MTRT_OK)
        return rc;
      int64_t rpp = rows_per_part;
      void *split_args[] = {&x, &d0, &d1, &nb, &rpp, &stage};
      rc = launch(st, KernelName("mtrt_amax_cols_split_") + u + xn, uint32_t(blocks * parts), kBlock, as_hip(stream), split_args);
      if (rc != MTRT_OK)
        return rc;
      void *finish_args[] = {&stage, &count, &qmax, &amax_out, &scale_out};
      return launch(st, KernelName("mtrt_amax_finish_") + xn, blocks_for(count, kBlock), kBlock, as_hip(stream), finish_args);
    }
    if (blocks <= int64_t(kMaxGrid) * 1024)
      return launch(st, KernelName("mtrt_amax_cols_") + u + xn, uint32_t(blocks), kBlock, as_hip(stream), args);
  }
  return launch(st, KernelName("mtrt_amax_cols_any_") + xn, blocks_for((d0 / nb) * d1, kBlock), kBlock, as_hip(stream), args);
}

int32_t mtrt_hip_quantize(mtrt_stream_t stream, const void *x, int32_t x_dtype, void *q, int32_t q_dtype,
                          const float *scale, int32_t scale_kind, int64_t d0, int64_t d1, int64_t nb,
                          int32_t flags) {
  return qdq_dispatch(0, as_hip(stream), x, x_dtype, q, q_dtype, nullptr, scale, scale_kind, d0, d1, nb, flags);
}

int32_t mtrt_hip_dequantize(mtrt_stream_t stream, const void *q, int32_t q_dtype, void *y, int32_t y_dtype,
                            const float *scale, int32_t scale_kind, int64_t d0, int64_t d1, int64_t nb) {
  return qdq_dispatch(1, as_hip(stream), nullptr, y_dtype, const_cast<void *>(q), q_dtype, y, scale, scale_kind,
                      d0, d1, nb, 0);
}

int32_t mtrt_hip_quantize_dequantize(mtrt_stream_t stream, const void *x, int32_t x_dtype, void *q,
                                     int32_t q_dtype, void *y, const float *scale, int32_t scale_kind,
                                     int64_t d0, int64_t d1, int64_t nb, int32_t flags) {
  return qdq_dispatch(2, as_hip(stream), x, x_dtype, q, q_dtype, y, scale, scale_kind, d0, d1, nb, flags);
}

namespace {
std::atomic<int32_t> g_wait_limit{1 << 16};

// Highest and lowest element offset a [d0, d1] view with these strides touches, relative to its base.
bool view_extent(int64_t offset, int64_t d0, int64_t d1, int64_t s0, int64_t s1, int64_t *lo, int64_t *hi) {
  const __int128 a = __int128(d0 - 1) * s0, b = __int128(d1 - 1) * s1;
  const __int128 l = offset + (a < 0 ? a : 0) + (b < 0 ? b : 0), h = offset + (a > 0 ? a : 0) + (b > 0 ? b : 0);
  if (l < -(__int128(1) << 62) || h > (__int128(1) << 62))
    return false;
  *lo = int64_t(l);
  *hi = int64_t(h);
  return true;
}

int32_t view_dispatch(bool quantize, hipStream_t stream, const void *f, int32_t f_dtype, const mtrt_hip_view2d *fv, const void *q,
                      int32_t q_dtype, const mtrt_hip_view2d *qv, const float *scale, int32_t kind, int64_t d0, int64_t d1,
                      int64_t nb, int32_t flags) {
  clear_error();
  const char *xn = float_name(f_dtype);
  if (!xn)
    return set_error(MTRT_INVALID_ARGUMENT, "float operand dtype %d is not one of f32/f16/bf16", f_dtype);
  if (q_dtype != MTRT_I8 && q_dtype != MTRT_F8E4M3FN && q_dtype != MTRT_I4)
    return set_error(MTRT_INVALID_ARGUMENT, "views carry one code per byte (i8, f8E4M3FN, i4); dtype %d is packed or unknown", q_dtype);
  if (!fv || !qv)
    return set_error(MTRT_INVALID_ARGUMENT, "null view descriptor");
  if (d0 < 0 || d1 < 0)
    return set_error(MTRT_INVALID_ARGUMENT, "negative extent [%lld, %lld]", (long long)d0, (long long)d1);
  if (kind < MTRT_SCALE_UNIFORM || kind > MTRT_SCALE_COL)
    return set_error(MTRT_INVALID_ARGUMENT, "unknown scale kind %d", kind);
  if (kind != MTRT_SCALE_UNIFORM && nb <= 0)
    return set_error(MTRT_INVALID_ARGUMENT, "scale kind %d needs a positive scale count / block size, got %lld", kind, (long long)nb);
  if (kind == MTRT_SCALE_COL && d0 % nb != 0)
    return set_error(MTRT_INVALID_ARGUMENT, "block size %lld does not divide the blocked extent %lld", (long long)nb, (long long)d0);
  if (flags & ~(MTRT_Q_ROUND_TO_INT | MTRT_F8_REFHOST | MTRT_F8_VIA_F16) || ((flags & MTRT_F8_REFHOST) && (flags & MTRT_F8_VIA_F16)))
    return set_error(MTRT_INVALID_ARGUMENT, "bad flag bits 0x%x", flags);
  if (d0 == 0 || d1 == 0)
    return MTRT_OK;
  int64_t n;
  if (!element_count(d0, d1, &n) || n >= (int64_t(1) << 40))
    return set_error(MTRT_INVALID_ARGUMENT, "view of [%lld, %lld] elements is too large", (long long)d0, (long long)d1);
  if (!f || !q || !scale)
    return set_error(MTRT_INVALID_ARGUMENT, "null operand");
  if (!aligned(f, float_bytes(f_dtype)))
    return set_error(MTRT_INVALID_ARGUMENT, "float operand is not aligned to its element size");
  // a view must stay at or above its base pointer (the allocation starts there); its upper end is the caller's word
  int64_t lo, hi;
  if (!view_extent(fv->offset, d0, d1, fv->stride0, fv->stride1, &lo, &hi) || lo < 0 ||
      !view_extent(qv->offset, d0, d1, qv->stride0, qv->stride1, &lo, &hi) || lo < 0)
    return set_error(MTRT_INVALID_ARGUMENT, "view reaches below its base pointer or overflows 62-bit offsets");
  DeviceState *st = device_state();
  if (!st)
    return MTRT_RUNTIME_ERROR;
  if (kind == MTRT_SCALE_UNIFORM)
    nb = 1;
  int64_t fo = fv->offset, fs0 = fv->stride0, fs1 = fv->stride1, qo = qv->offset, qs0 = qv->stride0, qs1 = qv->stride1;
  if (fs1 == 1 && qs1 == 1 && (d0 == 1 || (fs0 == d1 && qs0 == d1))) {
    // Dense in both operands (what a launch with whole row-major tensors passes): the contiguous entry points' own
    // dispatch on the offset pointers, tile kernels when aligned (f16 [8192, 8192] to i8: 56 us row by row, 41 us so).
    void *fp = const_cast<char *>(static_cast<const char *>(f)) + fo * float_bytes(f_dtype);
    void *qp = const_cast<char *>(static_cast<const char *>(q)) + qo;
    if (quantize)
      return qdq_dispatch(0, stream, fp, f_dtype, qp, q_dtype, nullptr, scale, kind, d0, d1, nb, flags);
    return qdq_dispatch(1, stream, nullptr, f_dtype, qp, q_dtype, fp, scale, kind, d0, d1, nb, flags);
  }
  if (fs1 == 1 && qs1 == 1) {
    // Rows that are contiguous in both operands (row and column slices of row-major tensors, offset sub-tensors): the
    // row-walking kernels of the contiguous entry points, with the views' row strides as pitches (f16 [8192, 8192]
    // column slice: 1.3 TB/s one element per lane).  A per-tensor scale is the row kind with one scale.
    const int group = f_dtype == MTRT_F32 ? 4 : 8;
    const int32_t rkind = kind == MTRT_SCALE_COL ? MTRT_SCALE_COL : MTRT_SCALE_ROW;
    const void *fp = static_cast<const char *>(f) + fo * float_bytes(f_dtype);
    const void *qp = static_cast<const char *>(q) + qo;
    KernelName rname(quantize ? "mtrt_q_" : "mtrt_dq_");
    rname + (rkind == MTRT_SCALE_COL ? "colu_" : "rowu_") + xn + "_" + code_name(q_dtype);
    const int64_t chunks = std::max<int64_t>(1, (d1 / group + 63) / 64);
    const uint32_t rgrid = blocks_for(d0 * chunks, kBlock / 64);
    if (quantize) {
      void *rargs[] = {&fp, &qp, &scale, &n, &d1, &nb, &fs0, &qs0, &flags};
      return launch(st, rname, rgrid, kBlock, stream, rargs);
    }
    void *rargs[] = {&qp, &fp, &scale, &n, &d1, &nb, &fs0, &qs0};
    return launch(st, rname, rgrid, kBlock, stream, rargs);
  }
  // An operand that runs fastest along its first dimension (a transpose): 64 x 64 tiles through LDS, each side walked
  // along its own grain.  Otherwise one element per lane.
  auto magnitude = [](int64_t v) { return v < 0 ? -v : v; };
  const bool tiled = magnitude(fs0) < magnitude(fs1) || magnitude(qs0) < magnitude(qs1);
  KernelName name(quantize ? (tiled ? "mtrt_q_viewt_" : "mtrt_q_view_") : (tiled ? "mtrt_dq_viewt_" : "mtrt_dq_view_"));
  name + xn + "_" + code_name(q_dtype);
  const uint32_t grid = tiled ? uint32_t(std::min<int64_t>(((d0 + 63) / 64) * ((d1 + 63) / 64), int64_t(kMaxGrid) * 1024))
                              : blocks_for(n, kBlock);
  if (quantize) {
    void *args[] = {&f, &fo, &d0, &d1, &fs0, &fs1, &q, &qo, &d0, &d1, &qs0, &qs1, &scale, &nb, &kind, &flags};
    return launch(st, name, grid, kBlock, stream, args);
  }
  void *args[] = {&q, &qo, &d0, &d1, &qs0, &qs1, &f, &fo, &d0, &d1, &fs0, &fs1, &scale, &nb, &kind};
  return launch(st, name, grid, kBlock, stream, args);
}
} // namespace

int32_t mtrt_hip_quantize_view(mtrt_stream_t stream, const void *x, int32_t x_dtype, const mtrt_hip_view2d *x_view, void *q,
                               int32_t q_dtype, const mtrt_hip_view2d *q_view, const float *scale, int32_t scale_kind,
                               int64_t d0, int64_t d1, int64_t nb, int32_t flags) {
  return view_dispatch(true, as_hip(stream), x, x_dtype, x_view, q, q_dtype, q_view, scale, scale_kind, d0, d1, nb, flags);
}

int32_t mtrt_hip_dequantize_view(mtrt_stream_t stream, const void *q, int32_t q_dtype, const mtrt_hip_view2d *q_view, void *y,
                                 int32_t y_dtype, const mtrt_hip_view2d *y_view, const float *scale, int32_t scale_kind,
                                 int64_t d0, int64_t d1, int64_t nb) {
  return view_dispatch(false, as_hip(stream), y, y_dtype, y_view, q, q_dtype, q_view, scale, scale_kind, d0, d1, nb, 0);
}

int32_t mtrt_hip_set_wait_limit(int32_t polls) {
  return g_wait_limit.exchange(polls < 0 ? 0 : polls);
}

int32_t mtrt_hip_dynamic_quantize_dequantize(mtrt_stream_t stream, const void *x, int32_t x_dtype, void *q, int32_t q_dtype,
                                             void *y, int64_t n, float qmax, float *amax_out, float *scale_out,
                                             int32_t flags) {
  clear_error();
  const char *xn = float_name(x_dtype);
  if (!xn)
    return set_error(MTRT_INVALID_ARGUMENT, "float operand dtype %d is not one of f32/f16/bf16", x_dtype);
  if (q_dtype != MTRT_I8 && q_dtype != MTRT_F8E4M3FN)
    return set_error(MTRT_INVALID_ARGUMENT, "dynamic per-tensor quantization targets i8 or f8E4M3FN, got dtype %d", q_dtype);
  if (n < 0)
    return set_error(MTRT_INVALID_ARGUMENT, "negative element count %lld", (long long)n);
  if (n > 0 && (!x || !q))
    return set_error(MTRT_INVALID_ARGUMENT, "null operand");
  if (!scale_out)
    return set_error(MTRT_INVALID_ARGUMENT, "scale_out must point at device memory for one f32 (the quantize step reads the scale there)");
  if (flags & ~(MTRT_Q_ROUND_TO_INT | MTRT_F8_REFHOST | MTRT_F8_VIA_F16))
    return set_error(MTRT_INVALID_ARGUMENT, "unknown flag bits 0x%x", flags);
  DeviceState *st = device_state();
  if (!st)
    return MTRT_RUNTIME_ERROR;
  const int group = x_dtype == MTRT_F32 ? 4 : 8;
  // one workgroup per compute unit at most, and one slot of the exchange per workgroup (256 of them)
  const int64_t nvec = n / group, units = std::min(num_compute_units(st), 256);
  // (The 16-vector form of the 16-bit -> f8 pairs does not fit the 128 registers a lane of a 1024-lane workgroup has
  // and would keep some of the row in scratch memory; a kernel that needs more than a little scratch pays some 10 us
  // per launch for its allocation, more than the second launch costs, so those pairs stop at 4 vectors per lane.)
  const int max_nv = group == 8 && q_dtype == MTRT_F8E4M3FN ? 4 : 16;
  const bool one_launch = n > 0 && n % group == 0 && aligned(x, 16) && aligned(q, group) && (!y || aligned(y, 16)) &&
                          nvec <= units * 1024 * max_nv && !((flags & MTRT_F8_REFHOST) && (flags & MTRT_F8_VIA_F16));
  if (one_launch) {
    uint32_t *slot = reduction_slot(st, as_hip(stream));
    if (!slot)
      return MTRT_RUNTIME_ERROR;
    const int nv = nvec <= units * 1024 * 4 ? 4 : 16;
    const uint32_t grid = uint32_t((nvec + int64_t(1024) * nv - 1) / (int64_t(1024) * nv));
    int32_t limit = g_wait_limit.load();
    void *args[] = {&x, &q, &y, &n, &qmax, &amax_out, &scale_out, &slot, &flags, &limit};
    return launch(st, KernelName("mtrt_dynqdq_") + xn + "_" + code_name(q_dtype) + "_v" + nv, grid, 1024,
                  as_hip(stream), args);
  }
  // Does not fit in the registers of one grid (or is not vector-aligned): the reduction, then the element-wise pass.
  const int32_t st1 = mtrt_hip_amax(stream, x, x_dtype, n, qmax, amax_out, scale_out);
  if (st1 != MTRT_OK)
    return st1;
  if (y)
    return qdq_dispatch(2, as_hip(stream), x, x_dtype, q, q_dtype, y, scale_out, MTRT_SCALE_UNIFORM, 1, n, 1, flags);
  return qdq_dispatch(0, as_hip(stream), x, x_dtype, q, q_dtype, nullptr, scale_out, MTRT_SCALE_UNIFORM, 1, n, 1, flags);
}

int32_t mtrt_hip_dynamic_quantize_rows(mtrt_stream_t stream, const void *x, int32_t x_dtype, void *q, int32_t q_dtype,
                                       int64_t rows, int64_t d, float qmax, float *amax_out, float *scale_out,
                                       int32_t flags) {
  clear_error();
  const char *xn = float_name(x_dtype);
  if (!xn)
    return set_error(MTRT_INVALID_ARGUMENT, "float operand dtype %d is not one of f32/f16/bf16", x_dtype);
  if (q_dtype != MTRT_I8 && q_dtype != MTRT_F8E4M3FN)
    return set_error(MTRT_INVALID_ARGUMENT, "dynamic per-row quantization targets i8 or f8E4M3FN, got dtype %d", q_dtype);
  if (rows < 0 || d < 0)
    return set_error(MTRT_INVALID_ARGUMENT, "negative extent [%lld, %lld]", (long long)rows, (long long)d);
  int64_t n;
  if (!element_count(rows, d, &n) || n >= (int64_t(1) << 35))
    return set_error(MTRT_INVALID_ARGUMENT, "[%lld, %lld] elements exceed the supported 2^35", (long long)rows, (long long)d);
  if (flags & ~(MTRT_Q_ROUND_TO_INT | MTRT_F8_REFHOST | MTRT_F8_VIA_F16))
    return set_error(MTRT_INVALID_ARGUMENT, "unknown flag bits 0x%x", flags);
  if ((flags & MTRT_F8_REFHOST) && (flags & MTRT_F8_VIA_F16))
    return set_error(MTRT_INVALID_ARGUMENT, "MTRT_F8_REFHOST and MTRT_F8_VIA_F16 name two different conversions; pass one");
  if (n == 0)
    return MTRT_OK;                                    // no row has an element: nothing is written
  if (!x || !q)
    return set_error(MTRT_INVALID_ARGUMENT, "null operand");
  if (!scale_out)
    return set_error(MTRT_INVALID_ARGUMENT, "scale_out must point at device memory for one f32 per row");
  if (!aligned(x, float_bytes(x_dtype)))
    return set_error(MTRT_INVALID_ARGUMENT, "float operand is not aligned to its element size");
  DeviceState *st = device_state();
  if (!st)
    return MTRT_RUNTIME_ERROR;
  // One launch while a row fits in the registers of a wave (up to 64 x 16 vectors) or of a workgroup's four waves
  // (up to 256 x 16 vectors): the row is read once.  Other rows (not whole vectors, operands off alignment, longer)
  // run as the two launches whose results this call is defined by.
  const int group = x_dtype == MTRT_F32 ? 4 : 8;
  const int64_t nvec = d / group;
  // A wave holds up to 8 vectors per lane, a workgroup's lanes up to 16; the 16-bit -> f8 pairs stop at 8 (their
  // 16-vector form would spill to scratch memory, whose allocation costs a launch some 10 us).
  const int max_group_nv = group == 8 && q_dtype == MTRT_F8E4M3FN ? 8 : 16;
  if (d % group == 0 && aligned(x, 16) && aligned(q, group) && nvec <= 256 * max_group_nv) {
    // A wave per row while that fills the chip (at least four waves per SIMD); with fewer rows the four waves of a
    // workgroup share each row, which puts four times the waves on the same loads (f16 [2048, 4096] 8.5 -> 7.5 us,
    // [4096, 4096] 12.7 -> 11.8 us; [8192, 4096] 22.7 against 23.4 us the other way).  Rows shorter than one vector
    // per lane of a workgroup stay with the wave form.
    const bool few_rows = rows <= int64_t(16) * num_compute_units(st) && nvec >= 256;
    const bool per_wave = nvec <= 64 * 8 && !few_rows;
    const int64_t lanes = per_wave ? 64 : 256;
    int nv = 1;
    while (lanes * nv < nvec)
      nv *= 2;
    const int64_t grid = per_wave ? (rows + 3) / 4 : rows;
    if (grid <= int64_t(kMaxGrid)) {
      void *args[] = {&x, &q, &rows, &d, &qmax, &amax_out, &scale_out, &flags};
      return launch(st, KernelName("mtrt_dynq_rows_") + xn + "_" + code_name(q_dtype) + (per_wave ? "_v" : "_g4v") + nv,
                    uint32_t(grid), kBlock, as_hip(stream), args);
    }
  }
  const int32_t st1 = mtrt_hip_amax_scales(stream, x, x_dtype, MTRT_SCALE_ROW, rows, d, rows, qmax, amax_out, scale_out);
  if (st1 != MTRT_OK)
    return st1;
  return qdq_dispatch(0, as_hip(stream), x, x_dtype, q, q_dtype, nullptr, scale_out, MTRT_SCALE_ROW, rows, d, rows, flags);
}

namespace {
int32_t nvfp4_dispatch(bool quantize, hipStream_t stream, const void *xy, int32_t dtype, const void *q, const void *scales,
                       const float *tensor_amax, int64_t d0, int64_t d1, int32_t block_axis) {
  clear_error();
  const char *xn = float_name(dtype);
  if (!xn)
    return set_error(MTRT_INVALID_ARGUMENT, "float operand dtype %d is not one of f32/f16/bf16", dtype);
  if (d0 < 0 || d1 < 0)
    return set_error(MTRT_INVALID_ARGUMENT, "negative extent [%lld, %lld]", (long long)d0, (long long)d1);
  if (block_axis != 0 && block_axis != 1)
    return set_error(MTRT_INVALID_ARGUMENT, "invalid axis! Axis can be either last (1) or second last (0) dimension of the [d0, d1] view, got %d",
                     block_axis);
  int64_t n;
  if (!element_count(d0, d1, &n) || n >= (int64_t(1) << 40))
    return set_error(MTRT_INVALID_ARGUMENT, "tensor of [%lld, %lld] elements is too large", (long long)d0, (long long)d1);
  const int64_t blocked = block_axis ? d1 : d0;
  if (blocked % 16 != 0)
    return set_error(MTRT_INVALID_ARGUMENT, "shape(input)[axis] must be divisible by 16, got %lld", (long long)blocked);
  if (d0 == 0 || d1 == 0)
    return MTRT_OK;
  if (!xy || !q || !scales || !tensor_amax)
    return set_error(MTRT_INVALID_ARGUMENT, "null operand");
  if (!aligned(xy, 16) || !aligned(q, 16) || !aligned(tensor_amax, 4) || !aligned(scales, 8))
    return set_error(MTRT_INVALID_ARGUMENT, "the float operand and the codes must be 16-byte aligned, the scales 8-byte aligned");
  DeviceState *st = device_state();
  if (!st)
    return MTRT_RUNTIME_ERROR;
  const int group = dtype == MTRT_F32 ? 4 : 8;
  if (block_axis == 0) {
    if (d1 % group != 0)
      return set_error(MTRT_INVALID_ARGUMENT, "blocks along the second-to-last axis need the last extent %% %d == 0, got %lld",
                       group, (long long)d1);
    const int64_t units = quantize ? (d0 / 16) * (d1 / group) : d0 * (d1 / group);
    if ((units + kBlock - 1) / kBlock > int64_t(kMaxGrid) * 1024)
      return set_error(MTRT_INVALID_ARGUMENT, "tensor of %lld elements is too large", (long long)n);
    if (quantize) {
      void *args[] = {&xy, &q, &scales, &tensor_amax, &d0, &d1};
      return launch(st, KernelName("mtrt_nvfp4_qc_") + xn, uint32_t((units + kBlock - 1) / kBlock), kBlock, stream, args);
    }
    void *args[] = {&q, &scales, &tensor_amax, &xy, &d0, &d1};
    const int64_t blocks = std::min<int64_t>((units + kBlock - 1) / kBlock, int64_t(num_compute_units(st)) * 64);
    return launch(st, KernelName("mtrt_nvfp4_dqc_") + xn, uint32_t(blocks), kBlock, stream, args);
  }
  int64_t nvec = n / group;
  const int64_t blocks = (nvec + 4 * 8 * 64 - 1) / (4 * 8 * 64);   // 4 waves x 8 trips x 64 lanes per workgroup
  if (blocks > int64_t(kMaxGrid) * 1024)
    return set_error(MTRT_INVALID_ARGUMENT, "tensor of %lld elements is too large", (long long)n);
  if (quantize) {
    void *args[] = {&xy, &q, &scales, &tensor_amax, &nvec};
    return launch(st, KernelName("mtrt_nvfp4_q_") + xn, uint32_t(blocks), kBlock, stream, args);
  }
  void *args[] = {&q, &scales, &tensor_amax, &xy, &nvec};
  return launch(st, KernelName("mtrt_nvfp4_dq_") + xn, uint32_t(blocks), kBlock, stream, args);
}
} // namespace

int32_t mtrt_hip_nvfp4_quantize(mtrt_stream_t stream, const void *x, int32_t x_dtype, void *q_packed, void *scales,
                                const float *tensor_amax, int64_t d0, int64_t d1, int32_t block_axis) {
  return nvfp4_dispatch(true, as_hip(stream), x, x_dtype, q_packed, scales, tensor_amax, d0, d1, block_axis);
}

int32_t mtrt_hip_nvfp4_dequantize(mtrt_stream_t stream, const void *q_packed, const void *scales,
                                  const float *tensor_amax, void *y, int32_t y_dtype, int64_t d0, int64_t d1,
                                  int32_t block_axis) {
  return nvfp4_dispatch(false, as_hip(stream), y, y_dtype, q_packed, scales, tensor_amax, d0, d1, block_axis);
}

int32_t mtrt_hip_layernorm(mtrt_stream_t stream, const void *x, const void *gamma, const void *beta, void *y,
                           int32_t dtype, int64_t rows, int64_t d, float eps) {
  clear_error();
  const char *xn = float_name(dtype);
  if (!xn)
    return set_error(MTRT_INVALID_ARGUMENT, "layernorm dtype %d is not one of f32/f16/bf16", dtype);
  if (rows < 0 || d < 0)
    return set_error(MTRT_INVALID_ARGUMENT, "negative extent [%lld, %lld]", (long long)rows, (long long)d);
  int64_t n;
  if (!element_count(rows, d, &n) || n >= (int64_t(1) << 40))
    return set_error(MTRT_INVALID_ARGUMENT, "[%lld, %lld] elements exceed the supported 2^40", (long long)rows, (long long)d);
  if (rows == 0 || d == 0)
    return MTRT_OK;
  if (!x || !gamma || !beta || !y)
    return set_error(MTRT_INVALID_ARGUMENT, "null operand");
  const int eb = float_bytes(dtype);
  if (!aligned(x, eb) || !aligned(y, eb) || !aligned(gamma, eb) || !aligned(beta, eb))
    return set_error(MTRT_INVALID_ARGUMENT, "operand is not aligned to its element size");
  DeviceState *st = device_state();
  if (!st)
    return MTRT_RUNTIME_ERROR;
  const int per_vec = 16 / eb;
  const bool vec_ok = d % per_vec == 0 && aligned(x, 16) && aligned(y, 16) && aligned(gamma, 16) && aligned(beta, 16);
  const int nv = vec_ok ? pick_nv(d / per_vec) : 0;
  int64_t rows_arg = rows, d_arg = d;
  float eps_arg = eps;
  void *args[] = {&x, &gamma, &beta, &y, &rows_arg, &d_arg, &eps_arg};
  // Rows of at most 32 vectors: 8, 16 or 32 lanes per row, several rows to a wave (whatever the alignment).
  if (d / per_vec <= 32 && rows <= kMaxRowsPerWaveKernels) {
    const int lanes = d / per_vec <= 8 ? 8 : (d / per_vec <= 16 ? 16 : 32);
    return launch(st, KernelName("mtrt_layernorm_") + xn + "_u" + lanes + "v1", blocks_for(rows, kBlock / lanes), kBlock, as_hip(stream), args);
  }
  if (nv && rows <= kMaxRowsPerWaveKernels) {
    // One wave per row.  The eight-vector kernel runs five waves per SIMD; when that leaves a second, partly
    // filled round and eight waves per SIMD would hold every row at once, its 64-register form is faster.
    const int64_t simds = int64_t(num_compute_units(st)) * 4;
    const bool resident = nv == 8 && rows > 5 * simds && rows <= 8 * simds;
    return launch(st, KernelName("mtrt_layernorm_") + xn + "_v" + nv + (resident ? "r" : ""),
                  blocks_for(rows, kBlock / 64), kBlock, as_hip(stream), args);
  }
  int threads, gnv;
  if (vec_ok && !nv && rows <= int64_t(kMaxGrid) * 1024 && pick_group(d / per_vec, &threads, &gnv))
    return launch(st, KernelName("mtrt_layernorm_") + xn + "_g" + threads + "v" + gnv, uint32_t(rows), uint32_t(threads),
                  as_hip(stream), args);
  // Row lengths that are not whole vectors, or operands that are not 16-byte aligned: the same two schemes with
  // 128-bit accesses at element alignment and the last d % per_vec elements of a row moved one by one.
  if (!vec_ok && d >= per_vec) {
    int rnv = pick_nv(d / per_vec);
    if (rnv && rows <= kMaxRowsPerWaveKernels) {
      rnv = unaligned_nv(dtype, rnv, 64, true);
      return launch(st, KernelName("mtrt_layernorm_") + xn + "_u64v" + rnv, blocks_for(rows, kBlock / 64), kBlock, as_hip(stream), args);
    }
    if (!rnv && rows <= int64_t(kMaxGrid) * 1024 && pick_group(d / per_vec, &threads, &gnv))
      return launch(st, KernelName("mtrt_layernorm_") + xn + "_u" + threads + "v" + unaligned_nv(dtype, gnv, threads, true), uint32_t(rows), uint32_t(threads),
                    as_hip(stream), args);
  }
  return launch(st, KernelName("mtrt_layernorm_") + xn + "_any",
                uint32_t(std::min<int64_t>(rows, int64_t(num_compute_units(st)) * 8)), kBlock, as_hip(stream), args);
}

int32_t mtrt_hip_softmax(mtrt_stream_t stream, const void *x, void *y, int32_t dtype, int64_t rows, int64_t d) {
  clear_error();
  const char *xn = float_name(dtype);
  if (!xn)
    return set_error(MTRT_INVALID_ARGUMENT, "softmax dtype %d is not one of f32/f16/bf16", dtype);
  if (rows < 0 || d < 0)
    return set_error(MTRT_INVALID_ARGUMENT, "negative extent [%lld, %lld]", (long long)rows, (long long)d);
  int64_t n;
  if (!element_count(rows, d, &n) || n >= (int64_t(1) << 40))
    return set_error(MTRT_INVALID_ARGUMENT, "[%lld, %lld] elements exceed the supported 2^40", (long long)rows, (long long)d);
  if (rows == 0 || d == 0)
    return MTRT_OK;
  if (!x || !y)
    return set_error(MTRT_INVALID_ARGUMENT, "null operand");
  const int eb = float_bytes(dtype);
  if (!aligned(x, eb) || !aligned(y, eb))
    return set_error(MTRT_INVALID_ARGUMENT, "operand is not aligned to its element size");
  DeviceState *st = device_state();
  if (!st)
    return MTRT_RUNTIME_ERROR;
  const int per_vec = 16 / eb;
  const bool vec_ok = d % per_vec == 0 && aligned(x, 16) && aligned(y, 16);
  const int nv = vec_ok ? pick_nv(d / per_vec) : 0;
  int64_t rows_arg = rows, d_arg = d;
  void *args[] = {&x, &y, &rows_arg, &d_arg};
  // Rows of at most 32 vectors: 8, 16 or 32 lanes per row, several rows to a wave (whatever the alignment).
  if (d / per_vec <= 32 && rows <= kMaxRowsPerWaveKernels) {
    const int lanes = d / per_vec <= 8 ? 8 : (d / per_vec <= 16 ? 16 : 32);
    return launch(st, KernelName("mtrt_softmax_") + xn + "_u" + lanes + "v1", blocks_for(rows, kBlock / lanes), kBlock, as_hip(stream), args);
  }
  if (nv && rows <= kMaxRowsPerWaveKernels)
    return launch(st, KernelName("mtrt_softmax_") + xn + "_v" + nv,
                  blocks_for(rows, kBlock / 64), kBlock, as_hip(stream), args);
  int threads, gnv;
  if (vec_ok && !nv && rows <= int64_t(kMaxGrid) * 1024 && pick_group(d / per_vec, &threads, &gnv))
    return launch(st, KernelName("mtrt_softmax_") + xn + "_g" + threads + "v" + gnv, uint32_t(rows), uint32_t(threads),
                  as_hip(stream), args);
  // Row lengths that are not whole vectors, or operands that are not 16-byte aligned: the same two schemes with
  // 128-bit accesses at element alignment and the last d % per_vec elements of a row moved one by one.
  if (!vec_ok && d >= per_vec) {
    int rnv = pick_nv(d / per_vec);
    if (rnv && rows <= kMaxRowsPerWaveKernels) {
      rnv = unaligned_nv(dtype, rnv, 64, false);
      return launch(st, KernelName("mtrt_softmax_") + xn + "_u64v" + rnv, blocks_for(rows, kBlock / 64), kBlock, as_hip(stream), args);
    }
    if (!rnv && rows <= int64_t(kMaxGrid) * 1024 && pick_group(d / per_vec, &threads, &gnv))
      return launch(st, KernelName("mtrt_softmax_") + xn + "_u" + threads + "v" + unaligned_nv(dtype, gnv, threads, false), uint32_t(rows), uint32_t(threads),
                    as_hip(stream), args);
  }
  return launch(st, KernelName("mtrt_softmax_") + xn + "_any",
                uint32_t(std::min<int64_t>(rows, int64_t(num_compute_units(st)) * 8)), kBlock, as_hip(stream), args);
}

int32_t mtrt_hip_gemm_w8a8_prepack(mtrt_stream_t stream, const void *w_kn, void *w_nk, int64_t K, int64_t N) {
  clear_error();
  if (K < 0 || N < 0 || K > kMaxMatrixExtent || N > kMaxMatrixExtent)
    return set_error(MTRT_INVALID_ARGUMENT, "extents [%lld, %lld] are negative or beyond 2^31 - 1", (long long)K, (long long)N);
  if (K == 0 || N == 0)
    return MTRT_OK;
  if (!w_kn || !w_nk)
    return set_error(MTRT_INVALID_ARGUMENT, "null operand");
  DeviceState *st = device_state();
  if (!st)
    return MTRT_RUNTIME_ERROR;
  const int64_t tiles = ((K + 63) / 64) * ((N + 63) / 64);
  if (tiles > int64_t(kMaxGrid) * 1024)
    return set_error(MTRT_INVALID_ARGUMENT, "weight matrix [%lld, %lld] is too large", (long long)K, (long long)N);
  void *args[] = {&w_kn, &w_nk, &K, &N};
  return launch(st, KernelName("mtrt_w8_prepack_kn_to_nk"), uint32_t(tiles), kBlock, as_hip(stream), args);
}

int32_t mtrt_hip_gemm_w8a8(mtrt_stream_t stream, const void *a, const void *w_nk, const float *a_scale,
                           const float *w_scale, void *y, int64_t M, int64_t K, int64_t N) {
  clear_error();
  if (M < 0 || K < 0 || N < 0)
    return set_error(MTRT_INVALID_ARGUMENT, "negative extent M=%lld K=%lld N=%lld", (long long)M, (long long)K,
                     (long long)N);
  if (M > kMaxMatrixExtent || K > kMaxMatrixExtent || N > kMaxMatrixExtent)
    return set_error(MTRT_INVALID_ARGUMENT, "matrix extents are limited to 2^31 - 1, got M=%lld K=%lld N=%lld", (long long)M,
                     (long long)K, (long long)N);
  if (M == 0 || N == 0)
    return MTRT_OK;
  if (!a_scale || !w_scale || !y || (K > 0 && (!a || !w_nk)))
    return set_error(MTRT_INVALID_ARGUMENT, "null operand");
  if (!aligned(y, 2))
    return set_error(MTRT_INVALID_ARGUMENT, "output is not aligned to its element size");
  DeviceState *st = device_state();
  if (!st)
    return MTRT_RUNTIME_ERROR;
  void *args[] = {&a, &w_nk, &a_scale, &w_scale, &y, &M, &K, &N};
  // The matrix-core kernel moves 128-byte K slices with 16-byte accesses.
  if (K > 0 && K % 128 == 0 && aligned(a, 16) && aligned(w_nk, 16) && M * K < (int64_t(1) << 32) &&
      N * K < (int64_t(1) << 32)) {
    // Up to 32 rows are bound by reading the weights once: one workgroup per 32 weight rows, its eight waves splitting K
    // and reading whole rows (3.4 TB/s of weights; the fragment-order entry point reaches 4).  A tile launch lasts
    // one 256-row tile's whole K loop per round whatever M is (about 8 us + 6 ns per k: M = 16, K = 4096, N = 11008
    // 32.7 us against 13.4; M = 32, K = N = 8192 57.1 against 18.6; M = 1, K = N = 4096 27.6 against 11.2), so it
    // only wins on very large weights.  33 to 64 rows take the form with two activation row tiles per weight fragment.
    const double tile_rounds = double(((N + 255) / 256 + num_compute_units(st) - 1) / num_compute_units(st));
    const double small_us = tuning::kRowsFixedUs + double(N) * double(K) / tuning::kRowsBytesPerUs;
    const double tile_us = (tuning::kTileFixedUs + tuning::kTileUsPerRowByte * double(K)) * tile_rounds;
    // 65 to 128 rows: four row tiles per weight fragment, one workgroup of four waves per compute unit at a time, so
    // the launch runs in rounds of about 3.7 ns per k (M = 128, K = N = 4096: 33 -> 18.4 us; K = N = 8192: 57 -> 30.7;
    // N = 11008 needs two rounds and equals the tile launch)
    const int64_t tiles32 = (N + 31) / 32;
    const double mid_us = tuning::kRows128FixedUs + tuning::kRows128UsPerRowByte * double(K) *
                                                        double((tiles32 + num_compute_units(st) - 1) / num_compute_units(st));
    if (M <= 64 ? small_us < tile_us : M <= 128 && mid_us < tile_us) {
      return launch(st, KernelName(M <= 32 ? "mtrt_gemm_w8a8_nk_rows32" : M <= 64 ? "mtrt_gemm_w8a8_nk_rows64" : "mtrt_gemm_w8a8_nk_rows128"),
                    uint32_t(std::min<int64_t>(tiles32, int64_t(kMaxGrid) * 1024)), M <= 64 ? 512 : 256, as_hip(stream), args);
    }
    // 256 x 256 tiles, one workgroup per compute unit at a time, N panels dealt round-robin to the
    // 8 XCDs (gemm_core.hpp), so each set of panels takes 8 * ceil(panels / 8) * tiles_m workgroup
    // ids.  The launch runs in rounds of one tile per unit; when the last round would use at most
    // half of the units (or the whole launch does), its panels are cut into 128-wide halves.
    const int64_t panels = (N + 255) / 256, tiles_m = (M + 255) / 256, units = num_compute_units(st);
    const int64_t tiles = panels * tiles_m, rest = tiles % units;
    int64_t full_panels = panels;
    if (tiles * 2 <= units)
      full_panels = 0;
    else if (rest > 0 && rest * 2 <= units)
      full_panels = panels - (rest + tiles_m - 1) / tiles_m;
    const int64_t half_panels = (N - full_panels * 256 + 127) / 128;
    const int64_t grid = 8 * ((full_panels * tiles_m + 7) / 8) + 8 * ((half_panels * tiles_m + 7) / 8);   // each kind dealt evenly to the XCDs
    if (grid <= int64_t(kMaxGrid) * 1024) {
      void *fast_args[] = {&a, &w_nk, &a_scale, &w_scale, &y, &M, &K, &N, &full_panels};
      return launch(st, KernelName("mtrt_gemm_w8a8_nk"), uint32_t(grid), kBlock, as_hip(stream), fast_args);
    }
  }
  if (K > 0) {
    // Any other K or alignment still goes to the matrix cores: 128 x 128 tiles with byte-aligned loads and a
    // zero-padded last k-step (M=4096 K=4100 N=11008: 1.2 s on the one-element-per-lane kernel below).
    const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
    return launch(st, KernelName("mtrt_gemm_w8a8_nk_edge"), uint32_t(std::min<int64_t>(tiles, int64_t(kMaxGrid) * 1024)), kBlock,
                  as_hip(stream), args);
  }
  return launch(st, KernelName("mtrt_gemm_w8a8_nk_any"), blocks_for(M * N, kBlock), kBlock, as_hip(stream), args);
}

int64_t mtrt_hip_gemm_w8a8_fragments_bytes(int64_t K, int64_t N) {
  if (K <= 0 || N <= 0 || K % 128 != 0 || K > kMaxMatrixExtent || N > kMaxMatrixExtent)
    return 0;
  return ((N + 31) / 32) * 32 * K;
}

int32_t mtrt_hip_gemm_w8a8_prepack_fragments(mtrt_stream_t stream, const void *w, int32_t w_is_nk, void *w_frag,
                                             int64_t K, int64_t N) {
  clear_error();
  if (K <= 0 || N <= 0 || K % 128 != 0 || K > kMaxMatrixExtent || N > kMaxMatrixExtent)
    return set_error(MTRT_INVALID_ARGUMENT, "fragment order needs positive extents below 2^31 and K %% 128 == 0, got K=%lld N=%lld",
                     (long long)K, (long long)N);
  if (!w || !w_frag)
    return set_error(MTRT_INVALID_ARGUMENT, "null operand");
  if (!aligned(w_frag, 16))
    return set_error(MTRT_INVALID_ARGUMENT, "fragment buffer must be 16-byte aligned");
  DeviceState *st = device_state();
  if (!st)
    return MTRT_RUNTIME_ERROR;
  const int64_t chunks = mtrt_hip_gemm_w8a8_fragments_bytes(K, N) / 16;
  void *args[] = {&w, &w_frag, &K, &N, &w_is_nk};
  return launch(st, KernelName("mtrt_w8_prepack_frag"), blocks_for(chunks, kBlock), kBlock, as_hip(stream), args);
}

int32_t mtrt_hip_gemm_w8a8_fragments(mtrt_stream_t stream, const void *a, const void *w_frag, const float *a_scale,
                                     const float *w_scale, void *y, int64_t M, int64_t K, int64_t N) {
  clear_error();
  if (M < 0 || K <= 0 || N < 0 || K % 128 != 0)
    return set_error(MTRT_INVALID_ARGUMENT, "fragment-order GEMM needs K %% 128 == 0 and non-negative extents, got M=%lld K=%lld N=%lld",
                     (long long)M, (long long)K, (long long)N);
  if (M > kMaxMatrixExtent || K > kMaxMatrixExtent || N > kMaxMatrixExtent)
    return set_error(MTRT_INVALID_ARGUMENT, "matrix extents are limited to 2^31 - 1, got M=%lld K=%lld N=%lld", (long long)M,
                     (long long)K, (long long)N);
  if (M == 0 || N == 0)
    return MTRT_OK;
  if (!a || !w_frag || !a_scale || !w_scale || !y)
    return set_error(MTRT_INVALID_ARGUMENT, "null operand");
  if (!aligned(y, 2) || !aligned(a, 16) || !aligned(w_frag, 16))
    return set_error(MTRT_INVALID_ARGUMENT, "a and w_frag must be 16-byte aligned, y 2-byte aligned");
  if (M * K >= (int64_t(1) << 32))
    return set_error(MTRT_INVALID_ARGUMENT, "activations of %lld bytes exceed the kernel's 32-bit offsets", (long long)(M * K));
  DeviceState *st = device_state();
  if (!st)
    return MTRT_RUNTIME_ERROR;
  if (M > 32 && M <= 128) {
    // 33 to 128 rows: a tile launch lasts one 256-row tile's whole K loop per round (about 5 us + 4 ns per k, and no less
    // than reading the weights at 4.5 TB/s) and is mostly padding.  The wave-private kernels of gemm_core::rows32 with the
    // weight fragments straight into registers read the weights once with two (up to 64 rows) or four row tiles per
    // fragment: 64 rows about 5 us + 1 us per 4 MB of weights (K = N = 4096: 17.1 -> 10.2 us, K = 11008, N = 4096
    // 34.1 -> 17.5, K = N = 8192 29.3 -> 19.0), 128 rows one workgroup per compute unit at a time, rounds of about
    // 3.2 ns per k (K = N = 4096: 21.6 -> 16.0 us, K = N = 8192 38.0 -> 27.1; N = 11008 needs two rounds, 30.5 us, and
    // stays on the tiles at 23.9).
    const int64_t tiles32 = (N + 31) / 32, units = num_compute_units(st);
    const double weights = double(N) * double(K);
    const double tile_us = std::max(tuning::kFragTileFixedUs + tuning::kFragTileUsPerK * double(K), weights / tuning::kFragTileBytesPerUs) *
                           double(((N + 255) / 256 + units - 1) / units);
    const double rows_us = M <= 64 ? tuning::kFragRowsFixedUs + weights / tuning::kRowsWideBytesPerUs
                                   : tuning::kRows128FixedUs + tuning::kFragRows128UsPerK * double(K) * double((tiles32 + units - 1) / units);
    if (rows_us < tile_us) {
      void *rargs[] = {&a, &w_frag, &a_scale, &w_scale, &y, &M, &K, &N};
      return launch(st, KernelName(M <= 64 ? "mtrt_gemm_w8a8_frag_rows64" : "mtrt_gemm_w8a8_frag_rows128"),
                    uint32_t(std::min<int64_t>(tiles32, int64_t(kMaxGrid) * 1024)), M <= 64 ? 512 : 256, as_hip(stream), rargs);
    }
  }
  if (M <= 32 && (M > 16 || 2 * ((N + 31) / 32) <= int64_t(num_compute_units(st)))) {
    // 17 to 32 rows, and fewer rows when at most half of the compute units would get a 32-column tile: the wave-private
    // kernel, eight waves splitting K (M = 32 at (K, N) = (11008, 4096) 18.6 -> 12.9 us, (4096, 11008) 14.3 -> 13.5,
    // (8192, 8192) 15.8 -> 14.9; M = 16 at (11008, 4096) 15.1 -> 11.7).  With more tiles and up to 16 rows the
    // four-wave kernel below with its hand-counted waits stays ahead (M = 1 at (4096, 11008): 10.7 against 12.5 us).
    const int64_t tiles32 = (N + 31) / 32;
    void *rargs[] = {&a, &w_frag, &a_scale, &w_scale, &y, &M, &K, &N};
    return launch(st, KernelName("mtrt_gemm_w8a8_frag_rows32"), uint32_t(std::min<int64_t>(tiles32, int64_t(kMaxGrid) * 1024)), 512,
                  as_hip(stream), rargs);
  }
  if (M <= 16) {
    // one workgroup per 32-column tile, its four waves splitting K; between one and two tiles per compute unit one
    // workgroup per unit instead, the first ones taking a second tile (as for the int4 weights)
    const int64_t tiles32 = (N + 31) / 32, cus = num_compute_units(st);
    const uint32_t grid = uint32_t(M > 8 && tiles32 > cus && tiles32 <= 2 * cus ? cus : tiles32);
    void *sargs[] = {&a, &w_frag, &a_scale, &w_scale, &y, &M, &K, &N};
    return launch(st, KernelName("mtrt_gemm_w8a8_small16"), grid, kBlock, as_hip(stream), sargs);
  }
  // Tiles and rounds as in mtrt_hip_gemm_w8a8: 256 x 256, one workgroup per compute unit at a time;
  // a last round that would use at most half of the units is cut into 128-wide half tiles.
  const int64_t panels = (N + 255) / 256, tiles_m = (M + 255) / 256, units = num_compute_units(st);
  const int64_t tiles = panels * tiles_m, rest = tiles % units;
  {
    // ... or 256 x 384 tiles (fewer bytes moved per MFMA, every weight fragment loaded once per workgroup) where their
    // rounds come out shorter
    const double rounds = tiles * 2 <= units ? 0.5 : double(tiles / units) + (rest == 0 ? 0.0 : rest * 2 <= units ? 0.5 : 1.0);
    const int64_t wide_tiles = ((N + 383) / 384) * tiles_m;
    const double wide_rounds = tuning::kW8WideRoundPerRound * double((wide_tiles + units - 1) / units);
    const int64_t wide_grid = 8 * ((wide_tiles + 7) / 8);
    if (wide_rounds < rounds && wide_grid <= int64_t(kMaxGrid) * 1024) {
      void *wargs[] = {&a, &w_frag, &a_scale, &w_scale, &y, &M, &K, &N};
      return launch(st, KernelName("mtrt_gemm_w8a8_frag_t256x384"), uint32_t(wide_grid), 256, as_hip(stream), wargs);
    }
  }
  int64_t full_panels = panels;
  if (tiles * 2 <= units)
    full_panels = 0;
  else if (rest > 0 && rest * 2 <= units)
    full_panels = panels - (rest + tiles_m - 1) / tiles_m;
  const int64_t half_panels = (N - full_panels * 256 + 127) / 128;
  const int64_t grid = 8 * ((full_panels * tiles_m + 7) / 8) + 8 * ((half_panels * tiles_m + 7) / 8);   // each kind dealt evenly to the XCDs
  if (grid > int64_t(kMaxGrid) * 1024)
    return set_error(MTRT_INVALID_ARGUMENT, "problem [%lld, %lld] needs too many tiles", (long long)M, (long long)N);
  void *args[] = {&a, &w_frag, &a_scale, &w_scale, &y, &M, &K, &N, &full_panels};
  return launch(st, KernelName("mtrt_gemm_w8a8_frag"), uint32_t(grid), 256, as_hip(stream), args);
}

int32_t mtrt_hip_linear_dense(mtrt_stream_t stream, const void *x, const void *w_nk, const void *bias, void *y,
                              int32_t dtype, int64_t M, int64_t K, int64_t N) {
  clear_error();
  const char *xn = float_name(dtype);
  if (!xn)
    return set_error(MTRT_INVALID_ARGUMENT, "dense linear dtype %d is not one of f32/f16/bf16", dtype);
  if (M < 0 || K < 0 || N < 0)
    return set_error(MTRT_INVALID_ARGUMENT, "negative extent M=%lld K=%lld N=%lld", (long long)M, (long long)K,
                     (long long)N);
  if (M > kMaxMatrixExtent || K > kMaxMatrixExtent || N > kMaxMatrixExtent)
    return set_error(MTRT_INVALID_ARGUMENT, "matrix extents are limited to 2^31 - 1, got M=%lld K=%lld N=%lld", (long long)M,
                     (long long)K, (long long)N);
  if (M == 0 || N == 0)
    return MTRT_OK;
  if (!y || (K > 0 && (!x || !w_nk)))
    return set_error(MTRT_INVALID_ARGUMENT, "null operand");
  const int eb = float_bytes(dtype);
  if (!aligned(x, eb) || !aligned(w_nk, eb) || !aligned(y, eb) || !aligned(bias, eb))
    return set_error(MTRT_INVALID_ARGUMENT, "operand is not aligned to its element size");
  DeviceState *st = device_state();
  if (!st)
    return MTRT_RUNTIME_ERROR;
  // Decode-sized calls are bound by reading the weights once: up to 32 rows take one workgroup per 32 weight rows, its
  // eight waves splitting K (f16 M = 16, K = 4096, N = 11008: 55 us on the tile loop, 23.3 so, 3.9 TB/s of weights; f32
  // 473 -> 50 us); 33 to 64 rows the form with two activation row tiles per weight fragment; the tile loop (about
  // 8 us + 6 ns per byte of a row, per round) only wins on very large weights.
  const bool whole_slices = K > 0 && (K * eb) % 128 == 0 && aligned(x, 16) && aligned(w_nk, 16);
  const double tile_us = (tuning::kTileFixedUs + tuning::kTileUsPerRowByte * double(K * eb)) *
                         double(((N + 255) / 256 + num_compute_units(st) - 1) / num_compute_units(st));
  const double small_us = tuning::kRowsFixedUs + double(N) * double(K * eb) / tuning::kRowsWideBytesPerUs;
  const int64_t tiles32 = (N + 31) / 32;
  // 65 to 128 rows: four row tiles per weight fragment, rounds of one workgroup per compute unit (3.7 ns per byte of a row);
  // f32 operands are bound by their matrix instructions there, which the tile loop is as well, at eight times the rows
  const double mid_us = tuning::kRows128FixedUs + tuning::kRows128UsPerRowByte * double(K * eb) *
                                                      double((tiles32 + num_compute_units(st) - 1) / num_compute_units(st));
  if (whole_slices && (M <= 64 ? small_us < tile_us : M <= 128 && (dtype == MTRT_F32 || mid_us < tile_us))) {
    void *rargs[] = {&x, &w_nk, &bias, &y, &M, &K, &N};
    return launch(st, KernelName(M <= 32 ? "mtrt_gemm_dense_rows32_" : M <= 64 ? "mtrt_gemm_dense_rows64_" : "mtrt_gemm_dense_rows128_") + xn,
                  uint32_t(std::min<int64_t>(tiles32, int64_t(kMaxGrid) * 1024)), M <= 64 ? 512 : 256, as_hip(stream), rargs);
  }
  if (K > 0 && (K * eb) % 128 == 0 && aligned(x, 16) && aligned(w_nk, 16) && M * K * eb < (int64_t(1) << 32) &&
      N * K * eb < (int64_t(1) << 32)) {
    // operands in whole 128-byte slices of K: the matrix-core tile loop (tiles and rounds as in
    // mtrt_hip_gemm_w8a8; f16 [2048, 4096] x [11008, 4096]: 3654 us on the FMA kernel below, f32 3835 us)
    const int64_t panels = (N + 255) / 256, tiles_m = (M + 255) / 256, units = num_compute_units(st);
    const int64_t tiles256 = panels * tiles_m, rest = tiles256 % units;
    int64_t full_panels = panels;
    if (tiles256 * 2 <= units)
      full_panels = 0;
    else if (rest > 0 && rest * 2 <= units)
      full_panels = panels - (rest + tiles_m - 1) / tiles_m;
    const int64_t half_panels = (N - full_panels * 256 + 127) / 128;
    const int64_t grid = 8 * ((full_panels * tiles_m + 7) / 8) + 8 * ((half_panels * tiles_m + 7) / 8);   // each kind dealt evenly to the XCDs
    if (grid <= int64_t(kMaxGrid) * 1024) {
      void *margs[] = {&x, &w_nk, &bias, &y, &M, &K, &N, &full_panels};
      return launch(st, KernelName("mtrt_gemm_dense_mfma_") + xn, uint32_t(grid), kBlock, as_hip(stream), margs);
    }
  }
  void *args[] = {&x, &w_nk, &bias, &y, &M, &K, &N};
  if (K > 0) {
    // any other K or alignment: 128 x 128 tiles with element-aligned loads and a zero-padded last k-step
    // (f16 [2048, 4100] x [11008, 4100]: 3761 us on the FMA kernel below)
    const int64_t edge_tiles = ((M + 127) / 128) * ((N + 127) / 128);
    return launch(st, KernelName("mtrt_gemm_dense_edge_") + xn, uint32_t(std::min<int64_t>(edge_tiles, int64_t(kMaxGrid) * 1024)),
                  kBlock, as_hip(stream), args);
  }
  const int64_t tiles = ((M + 63) / 64) * ((N + 63) / 64);
  if (tiles > int64_t(kMaxGrid) * 1024)
    return set_error(MTRT_INVALID_ARGUMENT, "problem [%lld, %lld] needs too many tiles", (long long)M, (long long)N);
  return launch(st, KernelName("mtrt_gemm_dense_") + xn, uint32_t(tiles), kBlock, as_hip(stream), args);
}

namespace {
// The re-laid weights hold two layouts back to back: fragment order for the 32 x 32 matrix-core tiles (per 32
// columns and 64 k: 64 lanes x 16 bytes) and, when K is a multiple of 128, strip order for the M <= 16 kernel
// (per 16 columns and 128 k: 64 lanes x 16 bytes).
int64_t w4_fragment_bytes(int64_t K, int64_t N) { return ((N + 31) / 32) * (K / 64) * 1024; }
int64_t w4_strip_bytes(int64_t K, int64_t N) { return K % 128 == 0 ? ((N + 15) / 16) * (K / 128) * 1024 : 0; }
} // namespace

int64_t mtrt_hip_gemm_w4a16_prepacked_bytes(int64_t K, int64_t N) {
  if (K <= 0 || N <= 0 || K % 64 != 0 || K > kMaxMatrixExtent || N > kMaxMatrixExtent)
    return 0;
  return w4_fragment_bytes(K, N) + w4_strip_bytes(K, N);
}

int32_t mtrt_hip_gemm_w4a16_prepack(mtrt_stream_t stream, const void *w_kn_packed, void *w_prepacked, int64_t K,
                                    int64_t N) {
  clear_error();
  if (K <= 0 || N <= 0 || K % 64 != 0 || K > kMaxMatrixExtent || N > kMaxMatrixExtent)
    return set_error(MTRT_INVALID_ARGUMENT, "prepack needs positive extents below 2^31 and K %% 64 == 0, got K=%lld N=%lld",
                     (long long)K, (long long)N);
  if (!w_kn_packed || !w_prepacked)
    return set_error(MTRT_INVALID_ARGUMENT, "null operand");
  if (!aligned(w_prepacked, 16))
    return set_error(MTRT_INVALID_ARGUMENT, "prepacked buffer must be 16-byte aligned");
  DeviceState *st = device_state();
  if (!st)
    return MTRT_RUNTIME_ERROR;
  const int64_t dwords = w4_fragment_bytes(K, N) / 4;
  void *args[] = {&w_kn_packed, &w_prepacked, &K, &N};
  const int32_t rc = launch(st, KernelName("mtrt_w4_prepack"), blocks_for(dwords, kBlock), kBlock, as_hip(stream), args);
  if (rc != MTRT_OK || w4_strip_bytes(K, N) == 0)
    return rc;
  void *strips = static_cast<char *>(w_prepacked) + w4_fragment_bytes(K, N);
  void *args2[] = {&w_kn_packed, &strips, &K, &N};
  return launch(st, KernelName("mtrt_w4_prepack_strips"), blocks_for(w4_strip_bytes(K, N) / 4, kBlock), kBlock, as_hip(stream), args2);
}

int32_t mtrt_hip_gemm_w4a16(mtrt_stream_t stream, const void *a, const void *w_kn_packed, const void *w_prepacked,
                            const void *scale, void *y, int64_t M, int64_t K, int64_t N, int64_t block) {
  clear_error();
  if (M < 0 || K < 0 || N < 0)
    return set_error(MTRT_INVALID_ARGUMENT, "negative extent M=%lld K=%lld N=%lld", (long long)M, (long long)K,
                     (long long)N);
  if (M > kMaxMatrixExtent || K > kMaxMatrixExtent || N > kMaxMatrixExtent)
    return set_error(MTRT_INVALID_ARGUMENT, "matrix extents are limited to 2^31 - 1, got M=%lld K=%lld N=%lld", (long long)M,
                     (long long)K, (long long)N);
  if (M == 0 || N == 0)
    return MTRT_OK;
  if (block <= 0 || (K > 0 && K % block != 0))
    return set_error(MTRT_INVALID_ARGUMENT, "block size %lld does not divide K=%lld", (long long)block, (long long)K);
  if (!y || (K > 0 && (!a || !scale)) || (!w_kn_packed && !w_prepacked && K > 0))
    return set_error(MTRT_INVALID_ARGUMENT, "null operand");
  if (!aligned(a, 2) || !aligned(y, 2) || !aligned(scale, 2))
    return set_error(MTRT_INVALID_ARGUMENT, "operand is not aligned to its element size");
  DeviceState *st = device_state();
  if (!st)
    return MTRT_RUNTIME_ERROR;
  const bool fast = w_prepacked && K > 0 && K % 64 == 0 && block % 64 == 0 && aligned(a, 16) && aligned(w_prepacked, 16);
  if (fast && M > 32 && M <= 64) {
    // Between 33 and 64 rows a 128-row tile is at least half padding and the launch lasts as long as one tile's K
    // loop; two launches of the small-M kernels (rows 0..31, then the rest; the second finds the weights in cache)
    // are shorter: M = 48 at (K, N) = (4096, 4096) 22.2 us as one tile launch, (11008, 4096) 52.0, (4096, 11008) 23.1.
    const int32_t rc = mtrt_hip_gemm_w4a16(stream, a, w_kn_packed, w_prepacked, scale, y, 32, K, N, block);
    if (rc != MTRT_OK)
      return rc;
    return mtrt_hip_gemm_w4a16(stream, static_cast<const char *>(a) + 32 * K * 2, w_kn_packed, w_prepacked, scale,
                               static_cast<char *>(y) + 32 * N * 2, M - 32, K, N, block);
  }
  if (fast) {
    void *args[] = {&a, &w_prepacked, &scale, &y, &M, &K, &N, &block};
    if (M <= 16 && K % 128 == 0 && block % 128 == 0) {
      // one workgroup per compute unit, each a strip of 16-column tiles over all of K (weights in strip order)
      const void *strips = static_cast<const char *>(w_prepacked) + w4_fragment_bytes(K, N);
      void *sargs[] = {&a, &strips, &scale, &y, &M, &K, &N, &block};
      const int64_t tiles = (N + 15) / 16;
      return launch(st, KernelName("mtrt_gemm_w4a16_strips16"), uint32_t(std::min<int64_t>(tiles, num_compute_units(st))), kBlock,
                    as_hip(stream), sargs);
    }
    if (M <= 32) {
      // one workgroup per 32-column tile; between one and two tiles per compute unit, one workgroup per
      // compute unit instead (the kernel then gives workgroup g the tiles g and g + grid, which share the
      // activations; measured: 6 % faster at M = 16, 21 % at M = 32, 3 % slower at M = 5)
      const int64_t tiles = (N + 31) / 32, cus = num_compute_units(st);
      const uint32_t grid = uint32_t(M > 8 && tiles > cus && tiles <= 2 * cus ? cus : tiles);
      return launch(st, KernelName(M <= 16 ? "mtrt_gemm_w4a16_skinny16" : "mtrt_gemm_w4a16_skinny"), grid, kBlock, as_hip(stream), args);
    }
    // 256 x 384 or 256 x 256 tiles (four waves) or 128 x 256 / 128 x 128 tiles (eight waves), one workgroup per compute unit at a time.  A
    // launch runs in rounds of one tile per unit; a full round of the large tile takes 3.25 times a full round of
    // the small one for four times the work, and a partly filled last round is shorter than a full one (fewer
    // units share the power budget): 0.56 + 0.44 f^2 of it at fill f (measured over M = 48 ... 4096 at (K, N) =
    // (4096, 4096), (4096, 11008), (11008, 4096), (8192, 8192), (5120, 13824), (4096, 14336), (8192, 28672),
    // (4096, 2048): the estimate picks the faster kernel in all but near-ties; 128 x 64 tiles were never ahead
    // by more than 1 % there and only serve matrices at most 64 columns wide).
    if (M * K * 2 < (int64_t(1) << 32)) {
      const int64_t units = num_compute_units(st);
      const int64_t panels = (N + 255) / 256, tiles_m = (M + 255) / 256, big_tiles = panels * tiles_m;
      const int64_t wide_panels = (N + 127) / 128, wide_m = (M + 127) / 128, wide_tiles = wide_panels * wide_m;
      auto rounds = [units](int64_t tiles) {
        const double f = double(tiles % units) / double(units);
        return double(tiles / units) + (tiles % units ? tuning::kW4PartialRoundBase + tuning::kW4PartialRoundSlope * f * f : 0.0);
      };
      // (grids: the tiles dealt evenly to the eight XCDs, gemm_core::tile_of_even)
      const int64_t big = 8 * ((big_tiles + 7) / 8), wide = 8 * ((wide_tiles + 7) / 8);
      const int64_t narrow = 8 * ((((N + 63) / 64) * wide_m + 7) / 8);
      const int64_t huge_tiles = ((N + 383) / 384) * tiles_m, huge = 8 * ((huge_tiles + 7) / 8);
      const int64_t mid_tiles = panels * wide_m, mid = 8 * ((mid_tiles + 7) / 8);   // 128 x 256
      const double big_cost = tuning::kW4BigRoundPerSmallRound * rounds(big_tiles);
      const double huge_cost = tuning::kW4BigRoundPerSmallRound * tuning::kW4WideRoundPerBigRound * rounds(huge_tiles);
      const double mid_cost = tuning::kW4Mid256RoundPerSmallRound * rounds(mid_tiles);
      const double small_cost = std::min(rounds(wide_tiles), mid_cost);
      if (huge_cost < big_cost && huge_cost < small_cost && huge <= int64_t(kMaxGrid) * 1024)
        return launch(st, KernelName("mtrt_gemm_w4a16_t256x384"), uint32_t(huge), 256, as_hip(stream), args);
      if (big_cost < small_cost && big <= int64_t(kMaxGrid) * 1024)
        return launch(st, KernelName("mtrt_gemm_w4a16_t256x256"), uint32_t(big), 256, as_hip(stream), args);
      if (mid_cost < rounds(wide_tiles) && N > 64 && mid <= int64_t(kMaxGrid) * 1024)
        return launch(st, KernelName("mtrt_gemm_w4a16_t128x256"), uint32_t(mid), 512, as_hip(stream), args);
      if (N <= 64 && narrow <= int64_t(kMaxGrid) * 1024)
        return launch(st, KernelName("mtrt_gemm_w4a16_t128x64"), uint32_t(narrow), kBlock, as_hip(stream), args);
      if (wide <= int64_t(kMaxGrid) * 1024)
        return launch(st, KernelName("mtrt_gemm_w4a16_t128x128"), uint32_t(wide), 512, as_hip(stream), args);
    }
  }
  if (!w_kn_packed)
    return set_error(MTRT_INVALID_ARGUMENT, "this shape needs the original packed weights (K=%lld block=%lld)",
                     (long long)K, (long long)block);
  void *args[] = {&a, &w_kn_packed, &scale, &y, &M, &K, &N, &block};
  if (K > 0) {
    // any block, K, N and alignment from the original nibbles, still on the matrix cores: 128 x 128 tiles whose
    // weight stage is dequantised in the kernel (M = 256, K = N = 4096, block 32: 3660 us on the kernel below)
    const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
    return launch(st, KernelName("mtrt_gemm_w4a16_edge"), uint32_t(std::min<int64_t>(tiles, int64_t(kMaxGrid) * 1024)), kBlock,
                  as_hip(stream), args);
  }
  return launch(st, KernelName("mtrt_gemm_w4a16_any"), blocks_for(M * N, kBlock), kBlock, as_hip(stream), args);
}

} // extern "C"
