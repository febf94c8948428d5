// mmt4d on the gfx950 matrix cores.
//
// Contract: include/iree_amd_uk.h (mirrors iree_uk_mmt4d,
// runtime/src/iree/builtins/ukernel/mmt4d.h:14-21 of the reference). This file
// serves the tile shapes the gfx950 tile-size query hands out: M0 = N0 = 32 and
// a K0 such that one lane's MFMA operand (16 bytes) is one contiguous piece of a
// tile row:
//
//   type            MFMA                         K per MFMA   K0 served
//   f16 x f16 -> f32  v_mfma_f32_16x16x32_f16        32         8, 16
//   bf16 x bf16 -> f32 v_mfma_f32_16x16x32_bf16      32         8, 16
//   s8 x s8 -> s32    v_mfma_i32_16x16x64_i8         64         16, 32
//   (s8 with a row-major left-hand side and K in whole 32s only: v_mfma_i32_32x32x32_i8, K 32)
//   f32 x f32 -> f32  4 x v_mfma_f32_32x32x2_f32      8          4, 8
//   f16 -> f16, bf16 -> bf16 (intermediate roundings skipped): as -> f32, rounded on store
//   e4m3 x e4m3 -> f32 v_mfma_scale_f32_32x32x64_f8f6f4  64         16
//   (f16 / bf16 with the fused SiLU epilogue: v_mfma_f32_32x32x16_*, K 16)
//
// An operand fragment is always 1 KiB: R rows (the instruction's block, 32 or
// 16) of 64 / R chunks of 16 bytes; lane l feeds row l % R, chunk l / R. A
// packed tile row holds K0 elements, i.e. one, two or four of those chunks'
// worth is spread over as many consecutive K tiles of the outer row, and the
// per-lane global offset follows from that (packed_lane_off below); the 64-lane
// 128-bit load then lands the fragment in LDS in lane order, so LDS reads are
// linear whatever K0 is. With K0 = the 16 bytes of one chunk (what the
// tile-size query answers for the 32-row shapes) the global addresses are
// linear too. The fp8 instruction takes 32 bytes per lane (k = 32 (l / 32) ..
// + 32 of row l % 32): four K0 = 16 tiles make one operand block of 2 KiB,
// moved as two 1 KiB halves in which lanes 0-31 fetch one whole tile and lanes
// 32-63 the tile two further on. (OCP e4m3fn, unit block scales.)
//
// Kernel shape: a workgroup of 2 x kWavesN waves (4 by default) owns a macro
// tile of (2*WM) x (kWavesN*WN) blocks of R x R; each wave accumulates WM x WN
// blocks in registers (a 128 x 128 tile for the large variant). The K loop
// moves operand fragments global -> LDS with direct-to-LDS 128-bit buffer loads
// (no register staging) into a ring of K-step slots, several K-steps ahead of
// the MFMAs; fragments are read from LDS one K-step ahead and every memory
// instruction is issued in the shadow of an MFMA. Workgroup ids are remapped so
// that the 8 XCDs (which receive consecutive workgroup ids round-robin) each
// work on a compact block of macro tiles and reuse operand panels in their own
// L2.
//
// Measured bound that matters more than the nominal peak: the matrix pipe is
// power-limited by operand toggling. With N(0,1) f16 operands a register-only
// loop of v_mfma_f32_32x32x16_f16 sustains 1.45-1.7 PFLOP/s on MI355X and one
// of v_mfma_f32_16x16x32_f16 1.8-1.9 (both 2.3-2.4 with all-zero operands),
// which is why f16 / bf16 run on the 16-row shape, and so does i8 (uniform
// random bytes: 3.47 POP/s with the 32-row instruction, 4.16 with the 16-row
// one). fp8 stays on 32x32x64: the 16-row shape is 8 % ahead there as well,
// but its K-step is 128 bytes of a row, which the LDS rings of the tiles that
// run two per compute unit cannot hold. The clock drops under that limit, so
// every stall cycle costs more time as well.
//
// This header holds the kernel itself (the body as a device function, so that
// the library's launcher and the code object built for a HAL executable can
// both wrap it in a __global__ of their own).
#ifndef IREE_AMD_UK_MMT4D_MFMA_KERNEL_H_
#define IREE_AMD_UK_MMT4D_MFMA_KERNEL_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "uk_fp8.h"
#include "uk_mfma_cfg.h"

namespace uk {

struct MfmaArgs {
  const char* lhs;  // offset applied
  const char* rhs;
  char* out;
  int64_t lhs_stride_bytes, rhs_stride_bytes, out_stride_bytes;
  int M, N;          // outer tile counts
  int ksteps;        // whole MFMA K-steps = K * K0 / kMfmaK
  int tail_tiles;    // K tiles left over after them (less than one MFMA's worth)
  int tiles_m, tiles_n;  // macro-tile grid
  int accumulate;
  // row-major result (mmt4d fused with the unpack that would follow it): the
  // matrix has out_rows x out_cols elements, out_stride_bytes is its row pitch
  int row_major_out, out_rows, out_cols;
  // row-major left-hand side (the pack of the LHS fused into the loads): lhs is
  // the out_rows x K matrix itself, lhs_stride_bytes its row pitch; the block
  // of (outer row i, K-step ks) is rows 32 i .. 32 i + 31, bytes
  // lhs_step_bytes * ks .. of each row
  int lhs_row_major;
  int k0_div;        // the instruction's K extent / K0: 1, 2 (or 4 for the 16-row shapes)
  // fused SiLU * up epilogue only: scales of the gate and up accumulators and
  // the inverse scale of the e4m3 result
  float gate_scale, up_scale, inv_out_scale;
  // row-major result of a float type only: factor applied on the store
  float out_scale;
  // K split (launch side): k_slices > 1 = workgroup row blockIdx.y computes
  // K-steps [y * slice_ksteps, ...) into the tiled partial result
  // out + y * slice_out_bytes
  int k_slices, slice_ksteps;
  int64_t slice_out_bytes;
  // batch (launch side): workgroup plane blockIdx.z multiplies the operands
  // that lie z * {lhs,rhs,out}_batch_bytes further on
  int batch;
  int64_t lhs_batch_bytes, rhs_batch_bytes, out_batch_bytes;
  // this many leading planes are dealt to the XCDs whole (see the __global__ wrapper)
  int batch_by_xcd;
  // the tiled result is larger than the L2s together: write it past the caches
  int stream_out;
  // macro-tile rows of one column panel of the workgroup order (see tile_coord)
  int panel_rows;
};

namespace {

constexpr int kPieceBytes = 1024;   // what one 64-lane 128-bit load moves


__device__ __forceinline__ void load_block_to_lds(__amdgpu_buffer_rsrc_t row, uint32_t lane_off,
                                                  uint32_t block_off, char* lds) {
  // 64 lanes x 16 bytes -> lds[0..1024) in lane order, from byte
  // block_off + lane_off of the operand row `row` describes. The row base and
  // block_off live in scalar registers and lane_off never changes, so a load
  // costs no per-lane address arithmetic.
  __builtin_amdgcn_raw_ptr_buffer_load_lds(row, (__attribute__((address_space(3))) void*)lds, 16,
                                           lane_off, block_off, 0, 0);
}

// Buffer descriptor of one operand row (its length is checked on the host).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t row_descriptor(const char* row) {
  return __builtin_amdgcn_make_buffer_rsrc((void*)row, 0, 0x7FFFFFFF, 0x00020000);
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Share of `n` items that falls to slot `i` of `slots` when they are spread evenly.
constexpr int share(int n, int slots, int i) { return (i + 1) * n / slots - i * n / slots; }

// Pins the issue order of one basic block to kMfma times {1 MFMA, its share of
// the kDsr LDS reads, its share of the kVmem vector-memory loads}. A memory
// instruction issued right behind an MFMA runs in its shadow; spreading them
// keeps a wave (which issues in order) from queueing behind a burst of loads
// while the matrix pipe runs dry. The LDS reads go behind the first kDsrMfma
// MFMAs only: the block that follows waits for the LAST read issued (LDS reads
// retire in order and the compiler waits for all of them), so the reads must
// be done while MFMAs of this block are still queued. The LDS reads and the
// direct-to-LDS loads must appear in the source in this same order: the
// compiler keeps their relative order (they may alias).
template <int kMfma, int kDsrMfma, int kDsr, int kVmem, int kInstrPerDsr, int I = 0>
__device__ __forceinline__ void spread_issue() {
  if constexpr (I < kMfma) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    if constexpr (I < kDsrMfma) {
      constexpr int d = share(kDsr, kDsrMfma, I) * kInstrPerDsr;
      if constexpr (d > 0) __builtin_amdgcn_sched_group_barrier(0x100, d, 0);
    }
    constexpr int v = share(kVmem, kMfma, I);
    if constexpr (v > 0) __builtin_amdgcn_sched_group_barrier(0x020, v, 0);
    spread_issue<kMfma, kDsrMfma, kDsr, kVmem, kInstrPerDsr, I + 1>();
  }
}

// Maps the hardware workgroup id to a macro-tile coordinate. Workgroup ids go
// round-robin over the 8 XCDs; give XCD x the x-th contiguous slice of the
// logical tile sequence, and order that sequence in column-panels of `kGroup`
// macro-tile rows so that a slice is a compact 2-D block. What an XCD's L2
// fetches for the r x c tiles it holds at a time is r tile heights of the
// left-hand side plus c tile widths of the right-hand side: 4 rows suit the
// square tile (32 resident per XCD: 4 x 8) and the tall one (64: 4 x 16 of
// 256 x 128), 8 rows the wide one (8 x 8 of 128 x 256; in panels of 4 rows
// every right-hand-side panel is fetched by twice as many XCD slices).
__device__ __forceinline__ void tile_coord(int bid, int tiles_m, int tiles_n, int kGroup,
                                           int* tm, int* tn) {
  constexpr int kXcds = 8;
  const int total = tiles_m * tiles_n;
  const int per = total / kXcds, rem = total % kXcds;
  const int xcd = bid % kXcds, idx = bid / kXcds;
  const int logical = xcd * per + (xcd < rem ? xcd : rem) + idx;
  const int group_size = kGroup * tiles_n;
  const int g = logical / group_size;
  const int first_m = g * kGroup;
  const int rows = (tiles_m - first_m) < kGroup ? (tiles_m - first_m) : kGroup;
  const int in_group = logical - g * group_size;
  *tm = first_m + in_group % rows;
  *tn = in_group / rows;
}

// K-loop organisation. LDS is a ring of kRing slots; slot (ks % kRing) holds
// K-step ks: the TM blocks of A followed by the TN blocks of B, 1 KiB each, in
// MFMA lane order. Waves synchronise once every kSync K-steps, at the start of
// the last K-step of a group: the barrier publishes the next group's data and
// frees the slots of the group just read. EVERY K-step then has the same
// memory work, spread evenly behind its MFMAs: the LDS reads of the next
// K-step's fragments, and this wave's share of the direct-to-LDS loads of the
// K-step that lies kRing - kSync + 1 ahead (into a slot the last barrier
// freed). Loads therefore stay in flight for kRing - 2 kSync + 1 K-steps.
// kSiluMul: instead of storing the accumulators, treat even outer columns as
// gate and the following odd ones as up, and store e4m3(silu(gate) * up) as
// left-hand-side tiles 32x16 of the next matmul (one byte per element).
// kForm: which of the operand forms the instance is compiled for: 0 = packed
// left-hand side, tiled result; 1 = row-major result; 2 = row-major left-hand
// side and result; 3 = row-major left-hand side, tiled result (the partial
// sums of a K split). (An instance compiled for one form has constant step sizes
// in its loop and one epilogue: measured 2 % (f16) to 6 % (i8) faster at 4096^3
// than one that reads the form from its arguments.)
// kStreamOut: the tiled result is not read again soon and may be written past
// the caches (off for the partial sums of a K split, which the reduction
// kernel reads next).
template <typename Cfg, int WM, int WN, int kRing, int kSync, bool kSiluMul = false, int kWavesN = 2,
          int kForm = 0, bool kStreamOut = true>
__device__ __forceinline__ void mmt4d_mfma_body(const MfmaArgs a, const int bid = blockIdx.x) {
  static_assert(kForm >= 0 && kForm <= 3 && (!kSiluMul || kForm == 0), "unknown operand form");
  constexpr bool lhs_row_major = kForm >= 2;
  constexpr bool row_major_out = kForm == 1 || kForm == 2;
  // kSwap: the MFMAs are issued with the operands exchanged (B fragment first),
  // so that a block's accumulator holds the TRANSPOSE in the instruction's
  // layout and a lane owns 4 consecutive COLUMNS of one row per register group
  // instead of 4 consecutive rows of one column. Row-major results then go out
  // (and come in) as 128-bit accesses and the SiLU form writes 4 bytes at a
  // time; measured 3 % faster at 4096^3 f16 for the row-major result. Tiled
  // results keep the instruction's own layout: there every 32-bit store
  // instruction already writes whole 128-byte lines, which measured 1-2 %
  // FASTER than 128-bit stores of quarter lines.
  constexpr bool kSwap = row_major_out || kSiluMul;
  typedef typename Cfg::frag_t frag_t;
  typedef typename Cfg::acc_t acc_t;
  typedef typename Cfg::out_t out_t;
  constexpr int kWaves = 2 * kWavesN;                // a 2 x kWavesN grid of waves
  // WM, WN, TM, TN count BLOCKS of R rows (R = 32 or 16: the instruction's
  // block); an outer tile of 32 rows is kPerTile of them.
  constexpr int R = Cfg::kRows, kPerTile = 32 / R;
  constexpr int kAccRegs = R * R / 64;               // accumulator registers of one block
  constexpr int kChunks = 64 / R;                    // 16-byte K chunks of a fragment row
  constexpr int TM = 2 * WM, TN = kWavesN * WN;      // blocks per workgroup
  static_assert(R == 32 || (R == 16 && Cfg::kSub == 1 && !kSiluMul), "unsupported block shape");
  static_assert(TM % kWaves == 0 && TN % kWaves == 0, "every wave loads whole operand rows");
  constexpr int kSub = Cfg::kSub;
  constexpr int kBlockBytes = kSub * kPieceBytes;   // one R-row operand block of one K-step
  constexpr int kABytes = TM * kBlockBytes;
  constexpr int kSlotBytes = (TM + TN) * kBlockBytes;
  constexpr int kAhead = kRing - kSync;
  constexpr int kARowsPerWave = TM / kWaves, kBRowsPerWave = TN / kWaves;
  constexpr int kLoadsPerStep = (kARowsPerWave + kBRowsPerWave) * kSub;  // per wave
  constexpr int kBody = (kSync % 2) ? 2 * kSync : kSync;        // K-steps per unrolled body
  constexpr int kFrags = WM + WN;               // operand fragments a wave reads per K-step
  constexpr int kPro = kRing - kSync + 1;       // K-steps loaded before the loop starts
  // MFMAs of a whole K-step / of the part behind a barrier, and how many of
  // them (from the front) get fragment reads slipped in behind them: the last
  // third or so stays free so that the reads have landed when the step ends.
  // kOuterB: with exchanged operands the MFMAs run over B blocks in the outer
  // loop, so that the instruction's first operand is the one that stays (and
  // the A fragments are the ones every first MFMA needs: they are read first).
  // Measured 2 % on the MLP block, 0.1-0.3 % on square problems.
  constexpr bool kOuterB = kSwap;
  constexpr int kOuter = kOuterB ? WN : WM, kInner = kOuterB ? WM : WN;
  constexpr int kMfmaAll = WM * WN, kMfmaRest = (kOuter - 1) * kInner;
  constexpr int kTail = kPerTile * kPerTile;    // (16-row shapes: 4x the MFMAs per K-step, each half as long)
  constexpr int kReadAll = kMfmaAll - (kMfmaAll >= 8 * kTail ? 6 * kTail : kMfmaAll / 2);
  constexpr int kReadRest = kMfmaRest - (kMfmaRest >= 8 * kTail ? 4 * kTail : kMfmaRest / 2);
  static_assert(kAhead >= kSync, "ring must hold two sync groups");
  static_assert(kPro >= kBody - 1, "the loop's remainder must already be in the ring");
  static_assert((kPro - kSync) * kLoadsPerStep < 64, "too many loads in flight for vmcnt");
  extern __shared__ __attribute__((aligned(1024))) char lds[];

  const int lane = threadIdx.x & 63;
  // fp8: the MFMA's block scales are register operands read from all lanes
  // whatever the execution mask; they are set here, where every lane is active
  // (a constant the compiler materialises inside a divergent region would
  // reach the active lanes only).
  int unit_scales = 0;
  if constexpr (Cfg::kSub == 2) unit_scales = Cfg::unit_scales();
  auto mfma = [&](const frag_t& x, const frag_t& y, const auto& c) {
    if constexpr (Cfg::kSub == 2) return Cfg::mfma(x, y, c, unit_scales);
    else return Cfg::mfma(x, y, c);
  };
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / kWavesN, wn = wave % kWavesN;
  int tm, tn;
  tile_coord(bid, a.tiles_m, a.tiles_n, a.panel_rows, &tm, &tn);
  const int i_base = tm * TM, j_base = tn * TN;
  const int T = a.ksteps;

  // Per-lane byte offset of a fragment inside the K-step of its outer row in
  // global memory. A lane feeds the instruction row l % R, 16-byte K chunk
  // l / R; a packed tile holds `cpt` chunks per row (K0 = the instruction's K
  // extent / k0_div), so chunk c lies in tile c / cpt at row pitch 16 cpt.
  // `sub` selects the block of R rows inside the 32-row tile. (fp8: two pieces
  // per lane, the second one 512-byte tile further.)
  const int frag_row = lane % R, frag_chunk = lane / R;
  const int cpt = kChunks / a.k0_div;
  auto packed_lane_off = [&](int sub) -> uint32_t {
    if constexpr (kSub == 2) return (lane >> 5) * 1024 + (lane & 31) * 16;
    return (uint32_t)((frag_chunk / cpt) * 512 * cpt + (sub * R + frag_row) * 16 * cpt +
                      (frag_chunk % cpt) * 16);
  };
  constexpr int kPieceStride = 512;
  constexpr int kStepBytes = kPerTile * kBlockBytes;   // of one outer row of packed tiles

  // Rows this wave copies: its share of the TM rows of A and TN of B. Out-of-range
  // rows are clamped to the last valid one (loaded, never stored).
  __amdgpu_buffer_rsrc_t a_src[kARowsPerWave], b_src[kBRowsPerWave];
  // Left-hand side: per-lane offset inside a row block, bytes between K-steps
  // and between the two pieces of a wide block. Packed: as the right-hand side.
  // Row-major: the load writes LDS in lane order, so which bytes a lane loads
  // decides where they lie. In the fragment's own lane order adjacent lanes
  // are adjacent ROWS, and a load instruction then looks up 64 different cache
  // lines where the packed form looks up 8. Instead 4 (2 where a K-step is 32
  // bytes of a row) adjacent lanes load the 16-byte chunks of ONE row's
  // K-step, 64 or 32 contiguous bytes, and a block lies in LDS row by row;
  // the chunks of a row are rotated by row / (rows per 256 bytes) so that the
  // 16 lanes of a fragment read that take one chunk of 16 consecutive rows
  // still hit every bank once. Two pieces per lane (fp8, a K-step is 64 bytes
  // of a row): piece j of a block holds rows 16 j .. 16 j + 15, all four
  // chunks of each, and a lane's two chunks (2 h and 2 h + 1 for K half h) are
  // read from the piece its row lies in.
  constexpr bool kLhsQuads = lhs_row_major;
  constexpr int kRowChunks = kChunks * kSub;          // 16-byte chunks of a row's K-step
  constexpr int kRotRows = 16 / kRowChunks;           // rows that share 256 bytes of LDS
  const int quad_row = lane / kRowChunks;             // (of the piece)
  const int quad_chunk = (lane % kRowChunks + 4 * kRowChunks - quad_row / kRotRows) % kRowChunks;
  auto lhs_read_off = [&](int chunk) -> uint32_t {
    if constexpr (kSub == 2) {
      const int q = frag_row % 16;
      return (uint32_t)((frag_row / 16) * kPieceBytes + q * 64 + ((chunk + q / 4) % 4) * 16);
    } else {
      return (uint32_t)(frag_row * 16 * kChunks + ((chunk + frag_row / kRotRows) % kChunks) * 16);
    }
  };
  const uint32_t a_read_off = !kLhsQuads ? (uint32_t)lane * 16 : lhs_read_off(frag_chunk * kSub);
  const uint32_t a_read_off_hi = !kLhsQuads ? (uint32_t)lane * 16 + kPieceBytes
                                            : kSub == 2 ? lhs_read_off(frag_chunk * kSub + 1) : 0u;
  uint32_t a_lane_off[kARowsPerWave][kSub], b_lane_off[kBRowsPerWave];
  const uint32_t a_step_bytes = lhs_row_major ? kChunks * 16 * kSub : kStepBytes;
#pragma unroll
  for (int r = 0; r < kARowsPerWave; ++r) {
    const int blk = i_base + wave * kARowsPerWave + r;
    int i = blk / kPerTile;
    const int sub = blk % kPerTile;
    i = i < a.M ? i : a.M - 1;
    if (lhs_row_major) {
      a_src[r] = row_descriptor(a.lhs);
#pragma unroll
      for (int j = 0; j < kSub; ++j) {
        int row = i * 32 + sub * R + j * 16 + quad_row;
        row = row < a.out_rows ? row : a.out_rows - 1;
        a_lane_off[r][j] = (uint32_t)row * (uint32_t)a.lhs_stride_bytes + quad_chunk * 16;
      }
    } else {
      a_src[r] = row_descriptor(a.lhs + (int64_t)i * a.lhs_stride_bytes);
#pragma unroll
      for (int j = 0; j < kSub; ++j) a_lane_off[r][j] = packed_lane_off(sub) + j * kPieceStride;
    }
  }
#pragma unroll
  for (int r = 0; r < kBRowsPerWave; ++r) {
    const int blk = j_base + wave * kBRowsPerWave + r;
    int j = blk / kPerTile;
    j = j < a.N ? j : a.N - 1;
    b_src[r] = row_descriptor(a.rhs + (int64_t)j * a.rhs_stride_bytes);
    b_lane_off[r] = packed_lane_off(blk % kPerTile);
  }
  // Accumulator layout of this lane inside a block. Instruction layout
  // (kSwap off): register v is row acc_row(v) = 8 (v / 4) + 4 (l / 32) + v % 4
  // (32x32) or 4 (l / 16) + v (16x16) of column acc_col = l % R. Exchanged
  // operands (kSwap on): the same with rows and columns swapped, i.e. row
  // acc_r = l % R and, for register group g (4 registers), the 4 columns from
  // acc_c0(g) on.
  auto acc_row = [&](int v) -> int {
    return R == 32 ? 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3) : 4 * (lane >> 4) + v;
  };
  const int acc_col = lane % R;
  constexpr int kGroups = kAccRegs / 4;
  const int acc_r = lane % R;
  auto acc_c0 = [&](int g) -> int { return R == 32 ? 8 * g + 4 * (lane >> 5) : 4 * (lane >> 4); };
  // 4 consecutive result elements; the buffers are only element-aligned.
  typedef out_t out4_t __attribute__((ext_vector_type(4), aligned(sizeof(out_t))));

  acc_t acc[WM][WN];
  // Initial accumulator values. Both variants run AFTER the first K-steps of
  // operand loads have been issued, in the shadow of their latency: reading the
  // result tile (accumulate flag) ...
  auto load_acc = [&]() {
    if constexpr (row_major_out) {
      // (rows and columns past the matrix edge are read from the last valid
      // one: their accumulators are never stored)
#pragma unroll
      for (int x = 0; x < WM; ++x) {
        int row = (i_base + wm * WM + x) * R + acc_r;
        row = row < a.out_rows ? row : a.out_rows - 1;
        const out_t* src = (const out_t*)(a.out + (int64_t)row * a.out_stride_bytes);
#pragma unroll
        for (int y = 0; y < WN; ++y)
#pragma unroll
          for (int g = 0; g < kGroups; ++g) {
            const int col = (j_base + wn * WN + y) * R + acc_c0(g);
            if (col + 4 <= a.out_cols) {
              const out4_t v4 = *(const out4_t*)(src + col);
#pragma unroll
              for (int e = 0; e < 4; ++e) acc[x][y][4 * g + e] = v4[e];
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const int c = col + e < a.out_cols ? col + e : a.out_cols - 1;
                acc[x][y][4 * g + e] = src[c];
              }
            }
          }
      }
    } else {
#pragma unroll
      for (int x = 0; x < WM; ++x)
#pragma unroll
        for (int y = 0; y < WN; ++y) {
          const int bi = i_base + wm * WM + x, bj = j_base + wn * WN + y;
          int i = bi / kPerTile, j = bj / kPerTile;
          i = i < a.M ? i : a.M - 1;
          j = j < a.N ? j : a.N - 1;
          const out_t* t = (const out_t*)(a.out + (int64_t)i * a.out_stride_bytes) + (int64_t)j * 1024 +
                           (bi % kPerTile) * R * 32 + (bj % kPerTile) * R;
#pragma unroll
          for (int v = 0; v < kAccRegs; ++v) acc[x][y][v] = t[acc_row(v) * 32 + acc_col];
        }
    }
  };
  // ... or clearing them.
  auto clear_acc = [&]() {
#pragma unroll
    for (int x = 0; x < WM; ++x)
#pragma unroll
      for (int y = 0; y < WN; ++y)
#pragma unroll
        for (int v = 0; v < kAccRegs; ++v) acc[x][y][v] = 0;
  };

  // Load `d` (of kLoadsPerStep) of this wave's share of K-step `ks` into ring
  // slot `slot`: its rows of A first, then its rows of B, kSub pieces each.
  auto issue_one = [&](int ks, int slot, int d) {
    char* base = lds + slot * kSlotBytes;
    const int r = d / kSub, j = d % kSub;
    if (r < kARowsPerWave) {
      load_block_to_lds(a_src[r], a_lane_off[r][j], (uint32_t)ks * a_step_bytes,
                        base + (wave * kARowsPerWave + r) * kBlockBytes + j * kPieceBytes);
    } else {
      const int rb = r - kARowsPerWave;
      load_block_to_lds(b_src[rb], b_lane_off[rb], (uint32_t)ks * kStepBytes + j * kPieceStride,
                        base + kABytes + (wave * kBRowsPerWave + rb) * kBlockBytes + j * kPieceBytes);
    }
  };
  auto issue_step = [&](int ks, int slot) {
#pragma unroll
    for (int d = 0; d < kLoadsPerStep; ++d) issue_one(ks, slot, d);
  };
  auto read_frag = [&](const char* p) -> frag_t {
    if constexpr (kSub == 1) {
      return *(const frag_t*)p;
    } else {
      const int4v lo = *(const int4v*)p, hi = *(const int4v*)(p + kPieceBytes);
      return frag_t{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    }
  };
  auto read_frag_at = [&](const char* block, uint32_t lo_off, uint32_t hi_off) -> frag_t {
    if constexpr (kSub == 1) {
      return *(const frag_t*)(block + lo_off);
    } else {
      const int4v lo = *(const int4v*)(block + lo_off), hi = *(const int4v*)(block + hi_off);
      return frag_t{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    }
  };
  // Fragment `r` (of kFrags) of this wave for the K-step in `slot`: its WN
  // blocks of B, then its WM blocks of A. The MFMAs run over A blocks in the
  // outer loop, so the fragments read last (A blocks 1..) are needed last.
  auto read_one = [&](int slot, int r, frag_t (&fa)[WM], frag_t (&fb)[WN]) {
    const char* s0 = lds + slot * kSlotBytes + lane * 16;
    // (the inner loop's operand first: all of it is needed by the first MFMAs)
    const bool is_b = kOuterB ? r >= WM : r < WN;
    const int idx = kOuterB ? (r < WM ? r : r - WM) : (r < WN ? r : r - WN);
    if (is_b) fb[idx] = read_frag(s0 + kABytes + (wn * WN + idx) * kBlockBytes);
    else fa[idx] = read_frag_at(lds + slot * kSlotBytes + (wm * WM + idx) * kBlockBytes, a_read_off, a_read_off_hi);
  };
  auto read_frags = [&](int slot, frag_t (&fa)[WM], frag_t (&fb)[WN]) {
#pragma unroll
    for (int r = 0; r < kFrags; ++r) read_one(slot, r, fa, fb);
  };
  // The memory work of one K-step, in the order spread_issue<nM, nR, ...> pins
  // it behind nM MFMAs: fragment reads of `read_slot` (behind the first nR
  // MFMAs), loads of K-step `ks`.
  auto memory_ops = [&](auto n_mfma, auto n_read_mfma, int ks, int load_slot, int read_slot,
                        frag_t (&na)[WM], frag_t (&nb)[WN]) {
    constexpr int nM = decltype(n_mfma)::value, nR = decltype(n_read_mfma)::value;
#pragma unroll
    for (int i = 0; i < nM; ++i) {
      if (i < nR) {
#pragma unroll
        for (int r = i * kFrags / nR; r < (i + 1) * kFrags / nR; ++r) read_one(read_slot, r, na, nb);
      }
#pragma unroll
      for (int d = i * kLoadsPerStep / nM; d < (i + 1) * kLoadsPerStep / nM; ++d)
        issue_one(ks, load_slot, d);
    }
  };
  // MFMAs of block rows [x0, x1) of this wave's WM x WN blocks.
  auto multiply_rows = [&](const frag_t (&fa)[WM], const frag_t (&fb)[WN], int o0, int o1) {
    if constexpr (kOuterB) {
      // exchanged operands: the B fragment is the instruction's first operand
      // and stays the same over the inner loop
#pragma unroll
      for (int y = 0; y < WN; ++y)
        if (y >= o0 && y < o1) {
#pragma unroll
          for (int x = 0; x < WM; ++x) acc[x][y] = mfma(fb[y], fa[x], acc[x][y]);
        }
    } else {
#pragma unroll
      for (int x = 0; x < WM; ++x)
        if (x >= o0 && x < o1) {
#pragma unroll
          for (int y = 0; y < WN; ++y) acc[x][y] = mfma(fa[x], fb[y], acc[x][y]);
        }
    }
  };
  auto multiply = [&](const frag_t (&fa)[WM], const frag_t (&fb)[WN]) {
    multiply_rows(fa, fb, 0, kOuter);
  };

  frag_t fa[2][WM], fb[2][WN];
  int done = 0;  // K-steps multiplied so far
  if (T > kRing) {
    // ---- pipelined path -------------------------------------------------
    int issue_ks = kPro, issue_slot = kPro % kRing;   // next K-step to load and its slot
    int read_slot = 0;                                // slot of K-step `done`
#pragma unroll 1
    for (int ks = 0; ks < kPro; ++ks) issue_step(ks, ks);
    if (a.accumulate) load_acc(); else clear_acc();
    wait_vmcnt<(kPro - kSync) * kLoadsPerStep>();  // the first kSync K-steps have landed
    __builtin_amdgcn_s_barrier();                  // (bare, as in the loop below)
    read_frags(0, fa[0], fb[0]);
    // Each body multiplies kBody K-steps (whole sync groups, and an even
    // number so that the fragment double buffer returns to fa[0]/fb[0]).
    while (done + kBody <= T) {
#pragma unroll
      for (int g = 0; g < kBody; ++g) {
        const int p = g & 1;
        const bool sync_point = (g % kSync) == kSync - 1;
        int next_slot = read_slot + 1; if (next_slot == kRing) next_slot = 0;
        // Past the end of K the last K-step is loaded again (into a slot nobody
        // reads any more): that keeps the number of loads in flight, and with
        // it the vmcnt arithmetic, constant.
        const int load_ks = issue_ks < T ? issue_ks : T - 1;
        if (!sync_point) {
          memory_ops(std::integral_constant<int, kMfmaAll>(), std::integral_constant<int, kReadAll>(),
                     load_ks, issue_slot, next_slot, fa[p ^ 1], fb[p ^ 1]);
          multiply(fa[p], fb[p]);
          spread_issue<kMfmaAll, kReadAll, kFrags, kLoadsPerStep, kSub>();
        } else {
          // The first row of MFMAs goes ahead of the barrier so that the
          // matrix pipe has work while the waves meet. This wave's reads of
          // K-steps <= done+g are complete once fa[p]/fb[p] have arrived, and
          // its loads of the next sync group once vmcnt has dropped to what
          // was issued since: the barrier then frees the slots of this group
          // and publishes the next group's data. The scheduling fences keep
          // the compiler from moving anything across the sequence.
          __builtin_amdgcn_sched_barrier(0);
          multiply_rows(fa[p], fb[p], 0, 1);
          __builtin_amdgcn_sched_barrier(0);
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
          wait_vmcnt<(kRing - 2 * kSync) * kLoadsPerStep>();
          // A bare barrier: __syncthreads() carries a release fence for which
          // the compiler drains every direct-to-LDS load still in flight.
          __builtin_amdgcn_s_barrier();
          __builtin_amdgcn_sched_barrier(0);
          memory_ops(std::integral_constant<int, kMfmaRest>(), std::integral_constant<int, kReadRest>(),
                     load_ks, issue_slot, next_slot, fa[p ^ 1], fb[p ^ 1]);
          multiply_rows(fa[p], fb[p], 1, kOuter);
          spread_issue<kMfmaRest, kReadRest, kFrags, kLoadsPerStep, kSub>();
          __builtin_amdgcn_sched_barrier(0);
        }
        ++issue_ks;
        ++issue_slot; if (issue_slot == kRing) issue_slot = 0;
        read_slot = next_slot;
      }
      done += kBody;
    }
    // Remainder (< kBody K-steps): everything has been issued; wait for all
    // of it and multiply straight out of the ring.
    wait_vmcnt<0>();
    __syncthreads();
#pragma unroll 1
    for (; done < T; ++done) {
      read_frags(read_slot, fa[0], fb[0]);
      multiply(fa[0], fb[0]);
      ++read_slot; if (read_slot == kRing) read_slot = 0;
    }
  } else {
    // ---- short-K path: everything fits in the ring ------------------------
#pragma unroll 1
    for (int ks = 0; ks < T; ++ks) issue_step(ks, ks);
    if (a.accumulate) load_acc(); else clear_acc();
    wait_vmcnt<0>();
    __syncthreads();
#pragma unroll 1
    for (; done < T; ++done) {
      read_frags(done, fa[0], fb[0]);
      multiply(fa[0], fb[0]);
    }
  }

  // K tail: fewer K tiles than one MFMA consumes are left. Their fragments
  // come straight from global memory, with zeros in the lanes (or lane halves)
  // that stand for the missing tiles.
  if (a.tail_tiles > 0) {
    const int64_t tail_off = (int64_t)T * kStepBytes;
    auto tail_frag = [&](const char* block, int sub) -> frag_t {
      const int4v zero = {0, 0, 0, 0};
      if constexpr (kSub == 1) {
        // (reached with a K0 below the instruction's K extent only: the lane's
        // chunk belongs to K tile chunk / cpt of the step)
        const int4v v = (frag_chunk / cpt) < a.tail_tiles ? *(const int4v*)(block + packed_lane_off(sub)) : zero;
        union { int4v i; frag_t f; } u;
        u.i = v;
        return u.f;
      } else {
        const int t0 = 2 * (lane >> 5);
        const char* p = block + (lane >> 5) * 1024 + (lane & 31) * 16;
        const int4v lo = t0 < a.tail_tiles ? *(const int4v*)p : zero;
        const int4v hi = t0 + 1 < a.tail_tiles ? *(const int4v*)(p + kPieceStride) : zero;
        return frag_t{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      }
    };
#pragma unroll
    for (int x = 0; x < WM; ++x) {
      const int blk = i_base + wm * WM + x;
      int i = blk / kPerTile;
      i = i < a.M ? i : a.M - 1;
      fa[0][x] = tail_frag(a.lhs + (int64_t)i * a.lhs_stride_bytes + tail_off, blk % kPerTile);
    }
#pragma unroll
    for (int y = 0; y < WN; ++y) {
      const int blk = j_base + wn * WN + y;
      int j = blk / kPerTile;
      j = j < a.N ? j : a.N - 1;
      fb[0][y] = tail_frag(a.rhs + (int64_t)j * a.rhs_stride_bytes + tail_off, blk % kPerTile);
    }
    multiply(fa[0], fb[0]);
    // (straight-line code whose results a row-major epilogue consumes under
    // per-lane row conditions)
    if constexpr (kSub == 2) {
#pragma unroll
      for (int x = 0; x < WM; ++x)
#pragma unroll
        for (int y = 0; y < WN; ++y) keep_result_in_all_lanes(acc[x][y]);
    }
  }

  // Epilogue. Tiled result (instruction layout): with 32x32 blocks one store
  // instruction writes two full 128-byte rows of the tile, with 16x16 blocks
  // four 64-byte row pieces. Row-major result (exchanged layout): every store
  // instruction writes 16 bytes per lane, 32 (or 16) rows of 32 (64) bytes.
  if constexpr (kSiluMul) {
    static_assert(WN % 2 == 0, "gate/up pairs must not straddle waves");
    // Block pair (y, y+1) -> 32x32 bytes, stored as the two 32x16 tiles
    // (rows of 16 bytes) that the next matmul reads as left-hand side: column
    // c of row r lies at (c / 16) * 512 + r * 16 + c % 16, so the 4 columns of
    // a register group are 4 consecutive bytes.
#pragma unroll
    for (int x = 0; x < WM; ++x)
#pragma unroll
      for (int y = 0; y < WN; y += 2) {
        const int i = i_base + wm * WM + x, j = j_base + wn * WN + y;
        if (i < a.M && j + 1 < a.N) {
          uint8_t* t = (uint8_t*)a.out + (int64_t)i * a.out_stride_bytes + (int64_t)(j >> 1) * 1024 + acc_r * 16;
          uint32_t w[kGroups];
#pragma unroll
          for (int g = 0; g < kGroups; ++g) {
            float h[4];
#pragma unroll
            for (int e = 0; e < 4; ++e)
              h[e] = silu_mul((float)acc[x][y][4 * g + e] * a.gate_scale,
                              (float)acc[x][y + 1][4 * g + e] * a.up_scale) * a.inv_out_scale;
            w[g] = pack4_e4m3(h[0], h[1], h[2], h[3]);
          }
          if constexpr (R == 32 && kGroups == 4) {
            // Group g of a lane is columns 8 g + 4 (l / 32) .. + 4 of row l % 32:
            // four pieces of 4 bytes, two in each of the two tiles. The lane
            // halves exchange them (v_permlane32_swap: lanes 32..63 of the
            // first register against lanes 0..31 of the second) so that lanes
            // 0..31 hold the 16 bytes of their row in the first tile and lanes
            // 32..63 those in the second: one 16-byte store instead of four of
            // 4 bytes (a compute unit takes a memory instruction only every
            // 30-50 cycles whatever it moves).
            const auto p = __builtin_amdgcn_permlane32_swap(w[0], w[2], false, false);
            const auto q = __builtin_amdgcn_permlane32_swap(w[1], w[3], false, false);
            typedef uint32_t row_t __attribute__((ext_vector_type(4)));
            const row_t row = {(uint32_t)p[0], (uint32_t)p[1], (uint32_t)q[0], (uint32_t)q[1]};
            *(row_t*)(t + (lane >> 5) * 512) = row;
          } else {
#pragma unroll
            for (int g = 0; g < kGroups; ++g) {
              const int c0 = acc_c0(g);
              *(uint32_t*)(t + (c0 >> 4) * 512 + (c0 & 15)) = w[g];
            }
          }
        }
      }
    return;
  }
  if constexpr (row_major_out) {
#pragma unroll
    for (int x = 0; x < WM; ++x) {
      const int row = (i_base + wm * WM + x) * R + acc_r;
      if (row < a.out_rows) {
        out_t* dst = (out_t*)(a.out + (int64_t)row * a.out_stride_bytes);
#pragma unroll
        for (int y = 0; y < WN; ++y)
#pragma unroll
          for (int g = 0; g < kGroups; ++g) {
            const int col = (j_base + wn * WN + y) * R + acc_c0(g);
            out4_t v4;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              if constexpr (std::is_floating_point<decltype(acc[x][y][0] + 0)>::value)
                v4[e] = (out_t)(acc[x][y][4 * g + e] * a.out_scale);   // (x 1.0f is exact)
              else
                v4[e] = acc[x][y][4 * g + e];
            }
            if (col + 4 <= a.out_cols) {
              *(out4_t*)(dst + col) = v4;
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (col + e < a.out_cols) dst[col + e] = v4[e];
            }
          }
      }
    }
    return;
  }
#pragma unroll
  for (int x = 0; x < WM; ++x)
#pragma unroll
    for (int y = 0; y < WN; ++y) {
      const int bi = i_base + wm * WM + x, bj = j_base + wn * WN + y;
      const int i = bi / kPerTile, j = bj / kPerTile;
      if (i < a.M && j < a.N) {
        out_t* t = (out_t*)(a.out + (int64_t)i * a.out_stride_bytes) + (int64_t)j * 1024 +
                   (bi % kPerTile) * R * 32 + (bj % kPerTile) * R;
        // 32-row blocks write whole 128-byte lines per instruction; a result
        // larger than the L2s goes past the caches (i8 4096^3: 65.3 -> 64.4 us,
        // fp8 56.65 -> 56.4); the 64-byte row pieces of 16-row blocks lose that
        // way (f16 110.4 -> 114.9; exchanging lane rows between the two blocks
        // of a tile first (v_permlane16_swap), so that they too write whole
        // lines past the caches, measured the same as their ordinary stores:
        // 103.8-104.7 against 104.4 us), and a small result is what the next
        // kernel reads.
        bool streamed = false;
        if constexpr (R == 32 && kStreamOut) {
          if (a.stream_out) {
            streamed = true;
#pragma unroll
            for (int v = 0; v < kAccRegs; ++v)
              __builtin_nontemporal_store((out_t)acc[x][y][v], &t[acc_row(v) * 32 + acc_col]);
          }
        }
        if (!streamed) {
#pragma unroll
          for (int v = 0; v < kAccRegs; ++v) t[acc_row(v) * 32 + acc_col] = acc[x][y][v];
        }
      }
    }
}

// LDS bytes a workgroup of the given shape needs (the dynamic shared memory of
// its launch).
template <typename Cfg, int WM, int WN, int kRing, int kWavesN = 2>
constexpr int mmt4d_mfma_lds_bytes() {
  return kRing * (2 * WM + kWavesN * WN) * Cfg::kSub * kPieceBytes;
}

}  // namespace
}  // namespace uk

#endif  // IREE_AMD_UK_MMT4D_MFMA_KERNEL_H_
