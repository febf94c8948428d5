// mmt4d for narrow left-hand sides (a matrix with fewer than 32 rows: the
// decode / GEMV shapes), on the matrix cores.
//
// The tile-size query narrows M0 to the next power of two that holds a static
// M below 32 (the reference does the same, compiler/src/iree/compiler/Codegen/
// Common/CPU/CPUMaterializeEncodingPass.cpp:343-353), so these calls arrive
// with M = 1 outer row of M0 x K0 tiles, N0 = 32 and a long right-hand side:
// the work is reading the right-hand side once, i.e. an HBM stream.
//
//   out[0][j][m0][n0] (+)= sum_k lhs[0][k][m0][k0] * rhs[j][k][n0][k0]
//
// A workgroup of 8 waves takes one outer column j at a time; wave w owns the
// w-th eighth of the K steps and keeps its part of the left-hand side in
// registers for the whole kernel, as the B operand of v_mfma_*_32x32 (column
// m0 of the block, zero beyond M0). The right-hand side streams through a
// rolling register buffer of 8 or 16 blocks of 1 KiB per wave (A operand: a packed
// tile is already in operand order), the request for block q+8 issued as block
// q is consumed, across tile boundaries, so the stream never drains. The 8
// partial 32x32 blocks are summed through LDS in wave order (deterministic)
// and rows m0 < M0 are stored.
//
// A narrow RIGHT-hand side (N0 < 32, M0 = 32, one outer column: a result with
// few columns, or the matrix-vector product) is the same problem with the
// operands exchanged: the reference turns a narrow-N result into a narrow-M one
// by transposition (compiler/src/iree/compiler/Codegen/Common/EncodingUtils.cpp:23-92
// and chooseMatmulTile, .../Common/CPU/CPUMaterializeEncodingPass.cpp:296-303).
// Here the kernel runs with the left-hand side streaming and the right-hand
// side in registers and stores every block transposed, as the 32 x N0 tile the
// caller asked for.
//
// The same kernel also serves the whole linear layer on a few rows
// (launch_matmul_rows_skinny: what iree_amd_uk_matmul_packed_rhs runs for a
// decode step): the left-hand side is then the row-major M x K matrix itself,
// whose rows take the place of the rows of the one narrow tile, and the result
// is written row by row (template switch kRows).
#include "uk_common.h"

#include <memory>
#include "uk_mfma_cfg.h"

#include <type_traits>

namespace uk {
namespace {

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
// right-hand-side blocks in flight per wave: 16 where a tile's steps are whole
// 16s, else 8 (N = 14336, K = 4096 f16: 22.84 -> 22.55 us at one row, 23.6 -> 23.1 at 8)
constexpr int kDepthMax = 16;

struct SkinnyArgs {
  const char* lhs;   // offsets applied
  const char* rhs;
  char* out;
  int64_t rhs_stride_bytes, out_stride_elems;  // per outer column j
  int N;             // outer columns
  int M0;
  int ksteps;        // MFMA K steps in total (the last one partial when tail_tiles > 0)
  // K tiles in the last step when K is not whole steps (0 = it is): the lanes
  // (or lane halves) that stand for the missing tiles of that step contribute
  // zeros on both sides (kTail kernels only)
  int tail_tiles;
  int steps_per_wave;
  int lhs_tile_bytes;  // M0 * K0 * element size
  int half_k0;
  int accumulate;
  // the block is stored transposed: element (m0, n0) of the kernel's M0 x 32
  // block at n0 * M0 + m0 (a 32 x M0 tile: the narrow right-hand side form)
  int transpose_out;
  // K split over workgroup rows: row blockIdx.y takes steps [y * chunk_steps,
  // ...) and writes its sums, in the accumulator's type, chunk_out_elems
  // further on (one launch row and chunk_steps = ksteps when K is not split)
  int chunk_steps;
  int64_t chunk_out_elems;
  // batch: workgroup plane blockIdx.z works on the operands that lie
  // z * {lhs,rhs,out}_batch_bytes further on (one plane and zeros without one)
  int batch;
  int64_t lhs_batch_bytes, rhs_batch_bytes, out_batch_bytes;
  // > 0: every wave fetches the left-hand side of its K slice (one contiguous
  // piece of the packed row) with direct-to-LDS loads of 1 KiB into its own
  // area of so many bytes of the dynamic LDS and reads its fragments from there
  int stage_wave_bytes;
  // > 0: the left-hand side is the row-major M0 x K matrix itself, rows so many
  // bytes apart (instead of one outer row of M0 x K0 tiles), and, with
  // out_row_pitch_elems > 0, the result the row-major M0 x out_cols matrix
  // (instead of N tiles of M0 x 32): the whole linear layer on a few rows.
  int64_t lhs_row_pitch_bytes;
  int64_t out_row_pitch_elems;
  int out_cols;
  // per-wave form with batch planes: plane z starts rot_tiles * z outer columns on
  int rot_tiles;
};

// SP: K steps per wave held in registers (compile-time bound; a.steps_per_wave <= SP).
// kPartialOut: the result is stored in the accumulator's type (the partial sums
// of a K split whose final result is narrower: f16, bf16).
// kPerWave: a K of at most SP (8 or 16) steps (the head size of an attention step, say)
// is not worth splitting over the waves: every wave takes all of K for an
// outer column of its own, 8 columns per workgroup at a time, and stores its
// block itself (no sum through LDS, no barrier).
// kRows: the row-major forms of left-hand side and result (SkinnyArgs); a
// compile-time switch so that the tile forms carry none of their address
// arithmetic (as a run-time one it cost the short-K batch form 16 %).
// kTail: K ends in a partial step (SkinnyArgs::tail_tiles); a kernel of its own so
// that whole-step calls carry none of its selects.
template <typename Cfg, int SP, bool kPartialOut = false, bool kPerWave = false, bool kRows = false,
          bool kTail = false>
__global__ __launch_bounds__(kThreads) void mmt4d_skinny_kernel(SkinnyArgs a) {
  static_assert(!(kTail && kRows), "the row-major forms take whole K steps only");
  typedef typename Cfg::frag_t frag_t;
  typedef typename Cfg::acc_t acc_t;
  typedef typename Cfg::out_t out_t;
  constexpr int kDepth = (SP % kDepthMax == 0) ? kDepthMax : 8;
  static_assert(SP % kDepth == 0, "the rolling buffer must divide the steps of a tile");
  // partial sums keep the accumulator's type (f32, or s32 for integer inputs)
  typedef typename std::conditional<std::is_same<out_t, int32_t>::value, int32_t, float>::type sum_t;
  typedef typename std::conditional<kPartialOut, sum_t, out_t>::type store_t;
  __shared__ sum_t partial[2][kWaves][16][64];
  // (fp8: the block scales of the MFMA, set while every lane is active)
  int unit_scales = 0;
  if constexpr (Cfg::kSub == 2) unit_scales = Cfg::unit_scales();
  a.lhs += blockIdx.z * a.lhs_batch_bytes;
  a.rhs += blockIdx.z * a.rhs_batch_bytes;
  a.out += blockIdx.z * a.out_batch_bytes;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int m0 = lane & 31, kh = lane >> 5;
  const int chunk_first = blockIdx.y * a.chunk_steps;
  const int chunk_end = chunk_first + a.chunk_steps < a.ksteps ? chunk_first + a.chunk_steps : a.ksteps;
  const int first = chunk_first + (kPerWave ? 0 : wave * a.steps_per_wave);
  int count = chunk_end - first;
  count = count < 0 ? 0 : (count > a.steps_per_wave ? a.steps_per_wave : count);

  // Right-hand side: lane offset inside an operand block (1 KiB; fp8: 2 KiB of
  // four K0 = 16 tiles, of which lanes 0..31 take tiles 0, 1 and lanes 32..63
  // tiles 2, 3 as two 16-byte pieces), block of (j, step).
  constexpr int kSub = Cfg::kSub;
  constexpr int kBlock = kSub * 1024;
  // Which columns a workgroup multiplies. The form that splits K over the waves
  // deals the 32 N columns to the workgroups of a launch row in units of 8, a
  // contiguous range of as equal a length as that allows each (448 outer
  // columns on 256 compute units: 56 columns each, where whole outer columns
  // were 1.75 a unit, paid as 2), and walks its range in windows of 32: lane
  // row n of a window at column c0 is column c0 + n, which may lie in the next
  // outer column (8 columns are whole cache lines of a K tile either way).
  // Columns past the range repeat its last column (the same bytes as a lane
  // that needs them: no further traffic) and their sums are not stored. The
  // per-wave form takes whole outer columns, one per wave.
  int c0, c_step, c_lim;
  if constexpr (kPerWave) {
    c0 = (blockIdx.x * kWaves + wave) * 32;
    c_step = gridDim.x * kWaves * 32;
    c_lim = a.N * 32;
  } else {
    // (workgroup ids go round-robin over the 8 XCDs: XCD x takes the x-th
    // contiguous slice of the ranges, so that neighbouring ranges, which share
    // the pair of cache lines at their boundary, meet in one L2)
    const int units = a.N * 4, groups = (int)gridDim.x;
    int bx;
    {
      const int per = groups / 8, more = groups % 8;
      const int xcd = (int)blockIdx.x % 8, idx = (int)blockIdx.x / 8;
      bx = xcd * per + (xcd < more ? xcd : more) + idx;
    }
    const int base = units / groups, rem = units - base * groups;
    const int u0 = bx * base + (bx < rem ? bx : rem);
    c0 = u0 * 8;
    c_step = 32;
    c_lim = (u0 + base + (bx < rem ? 1 : 0)) * 8;
  }
  // Batch planes of the per-wave form walk their outer columns from different
  // starting points: planes whose operands lie a power of two apart would
  // otherwise ask the same memory channels for the same offsets at the same time.
  const int rot = kPerWave && gridDim.z > 1 ? (int)(((int64_t)blockIdx.z * a.rot_tiles) % a.N) : 0;
  auto rotated = [&](int tile) -> int {
    tile += rot;
    return tile >= a.N ? tile - a.N : tile;
  };
  const char* const rhs_wave = a.rhs + (int64_t)(count > 0 ? first : 0) * kBlock;
  // this lane's piece of the first block of the window at column `at`
  auto window_ptr = [&](int at) -> const char* {
    int c = at + (lane & 31);
    c = c < c_lim ? c : c_lim - 1;
    c = c < a.N * 32 ? c : a.N * 32 - 1;        // (a window past the last one: any valid block)
    c = c < 0 ? 0 : c;
    const int r = c & 31;
    const int off = kSub == 2 ? ((lane >> 5) * 1024 + r * 16)
                    : a.half_k0 ? ((lane >> 5) * 512 + r * 16) : (r * 32 + (lane >> 5) * 16);
    return rhs_wave + (int64_t)(kPerWave ? rotated(c >> 5) : (c >> 5)) * a.rhs_stride_bytes + off;
  };
  const char* rhs_cur = window_ptr(c0);
  const char* rhs_next = window_ptr(c0 + c_step);
  // Partial last step: K tile of this lane's piece(s) inside a step (tiles are
  // 512 bytes of the right-hand side), whether the last step lacks it, and the
  // step of this wave's slice that is the last one of K (-1: another wave's).
  const int tile_lo = kSub == 2 ? 2 * (lane >> 5) : (lane >> 5), tile_hi = tile_lo + 1;
  const bool lo_missing = kTail && tile_lo >= a.tail_tiles, hi_missing = kTail && tile_hi >= a.tail_tiles;
  const int tail_s = kTail ? a.ksteps - 1 - (count > 0 ? first : 0) : -1;   // (of the blocks this wave loads)
  const bool owns_tail = tail_s >= 0 && tail_s < count;
  auto make_frag = [](int4v lo, int4v hi) -> frag_t {
    if constexpr (kSub == 2) {
      return frag_t{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    } else {
      union { int4v i; frag_t f; } u;
      u.i = lo;
      return u.f;
    }
  };
  // Steps past this wave's count still issue a load (of a valid block, so the
  // number of loads in flight stays constant) but contribute zeros, whatever
  // that block holds.
  auto load_block = [&](const char* window, int sp) -> frag_t {
    const int s = sp < count ? sp : 0;
    const char* p = window + (int64_t)s * kBlock;
    if constexpr (kTail) {
      // (a piece of a missing tile would lie past the end of the row: it is
      // fetched from the step's first tile instead and zeroed when consumed)
      const bool last = s == tail_s;
      const char* p_lo = p - (last && lo_missing ? tile_lo * 512 : 0);
      const char* p_hi = p + 512 - (last && hi_missing ? tile_hi * 512 : 0);
      const int4v lo = __builtin_nontemporal_load((const int4v*)p_lo);
      const int4v hi = kSub == 2 ? __builtin_nontemporal_load((const int4v*)p_hi) : lo;
      return make_frag(lo, hi);
    }
    // (non-temporal: the right-hand side is read once)
    const int4v lo = __builtin_nontemporal_load((const int4v*)p);
    const int4v hi = kSub == 2 ? __builtin_nontemporal_load((const int4v*)(p + 512)) : lo;
    return make_frag(lo, hi);
  };
  // (the zeroing happens when a block is consumed, not when it is requested:
  // touching the loaded registers earlier would wait for the load)
  auto live = [&](frag_t f, int sp) -> frag_t {
    const int4v zero = {0, 0, 0, 0};
    if constexpr (kTail) {
      if (sp == tail_s) {
        if constexpr (kSub == 2) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (lo_missing) f[e] = 0;
            if (hi_missing) f[4 + e] = 0;
          }
        } else {
          if (lo_missing) f = make_frag(zero, zero);
        }
      }
    }
    return sp >= count ? make_frag(zero, zero) : f;
  };

  // ---- the left-hand side and the first blocks of the first tile ------------
  frag_t ring[kDepth];
  frag_t xf[SP];
  // bytes of the packed left-hand side per K step: its K tiles are consecutive
  // (row-major: the bytes of one ROW per K step, 32, or 64 for fp8)
  constexpr bool rows_lhs = kRows;
  const int step_bytes = rows_lhs ? 32 * kSub : (kSub == 2 ? 4 : a.half_k0 ? 2 : 1) * a.lhs_tile_bytes;
  // this lane's first piece inside a step (the second one, fp8, a tile further;
  // row-major: the next 16 bytes of the row)
  const int piece_off = kSub == 2 ? 2 * kh * a.lhs_tile_bytes + m0 * 16
                        : a.half_k0 ? kh * a.lhs_tile_bytes + m0 * 16 : m0 * 32 + kh * 16;
  const int hi_off = rows_lhs ? 16 : a.lhs_tile_bytes;
  if (a.stage_wave_bytes > 0) {
    // Fetching the fragments straight into registers costs one load
    // instruction per K step and wave whatever M0 is (with M0 = 1 each moves
    // 32 bytes), and the compute unit takes a load instruction only every 30
    // cycles or so: 256 of them held the first tile up by 3 us. The slice is
    // contiguous in the packed row, so a few full-width loads bring it to LDS
    // (bytes past its end read as zeros: the descriptor ends there); the
    // right-hand side is requested right behind and only the slice is waited
    // for (loads return in order).
    extern __shared__ __attribute__((aligned(16))) char stage_all[];
    char* stage = stage_all + wave * a.stage_wave_bytes;
    // (a partial last step ends after its tail_tiles tiles: what lies beyond reads as zeros)
    const int slice = count * step_bytes - (owns_tail ? step_bytes - a.tail_tiles * a.lhs_tile_bytes : 0);
    // (row-major: the slice of every row, the rows SP steps and 16 bytes apart
    // in LDS so that the 16-byte reads of up to 16 rows touch every bank once;
    // a row's last load may run into the next row's place, which the next
    // row's loads, later in order, overwrite)
    const int row_stage = SP * step_bytes + 16;
    if (rows_lhs) {
#pragma unroll 1
      for (int r = 0; r < a.M0; ++r) {
        const __amdgpu_buffer_rsrc_t xsrc = __builtin_amdgcn_make_buffer_rsrc(
            (void*)(a.lhs + r * a.lhs_row_pitch_bytes + (int64_t)(count > 0 ? first : 0) * step_bytes), 0, slice,
            0x00020000);
#pragma unroll 1
        for (int off = 0; off < slice; off += 1024)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(
              xsrc, (__attribute__((address_space(3))) void*)(stage + r * row_stage + off), 16, lane * 16, off, 0, 0);
      }
    } else {
      const __amdgpu_buffer_rsrc_t xsrc = __builtin_amdgcn_make_buffer_rsrc(
          (void*)(a.lhs + (int64_t)(count > 0 ? first : 0) * step_bytes), 0, slice, 0x00020000);
#pragma unroll 1
      for (int off = 0; off < slice; off += 1024)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(xsrc, (__attribute__((address_space(3))) void*)(stage + off), 16,
                                                 lane * 16, off, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int d = 0; d < kDepth; ++d) ring[d] = load_block(rhs_cur, d);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kDepth * kSub) : "memory");
#pragma unroll
    for (int sp = 0; sp < SP; ++sp) {
      int4v lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
      if (m0 < a.M0 && sp < count) {
        const char* p = rows_lhs ? stage + m0 * row_stage + sp * step_bytes + kh * 16 * kSub
                                 : stage + sp * step_bytes + piece_off;
        // (LDS past the staged slice holds whatever was there: a missing tile is not read)
        if (!(sp == tail_s && lo_missing)) lo = *(const int4v*)p;
        if constexpr (kSub == 2) {
          if (!(sp == tail_s && hi_missing)) hi = *(const int4v*)(p + hi_off);
        }
      }
      xf[sp] = make_frag(lo, hi);
    }
  } else {
#pragma unroll
    for (int d = 0; d < kDepth; ++d) ring[d] = load_block(rhs_cur, d);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int sp = 0; sp < SP; ++sp) {
      const int s = first + (sp < count ? sp : 0);
      // K tile(s) of step s: two tiles of K0 = half the MFMA extent, or one;
      // fp8: four tiles, two per lane half.
      int4v lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
      if (m0 < a.M0 && sp < count) {
        const char* p = rows_lhs ? a.lhs + m0 * a.lhs_row_pitch_bytes + (int64_t)s * step_bytes + kh * 16 * kSub
                                 : a.lhs + (int64_t)s * step_bytes + piece_off;
        if (!(sp == tail_s && lo_missing)) lo = *(const int4v*)p;
        if constexpr (kSub == 2) {
          if (!(sp == tail_s && hi_missing)) hi = *(const int4v*)(p + hi_off);
        }
      }
      xf[sp] = make_frag(lo, hi);
    }
  }

  int parity = 0;
  for (; c0 < c_lim; c0 += c_step, parity ^= 1) {
    acc_t acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0;
#pragma unroll
    for (int sp = 0; sp < SP; ++sp) {
      if constexpr (Cfg::kSub == 2) acc = Cfg::mfma(live(ring[sp % kDepth], sp), xf[sp], acc, unit_scales);
      else acc = Cfg::mfma(live(ring[sp % kDepth], sp), xf[sp], acc);
      // refill the slot: kDepth steps ahead, wrapping into the next tile
      __builtin_amdgcn_sched_barrier(0);
      ring[sp % kDepth] = sp + kDepth < SP ? load_block(rhs_cur, sp + kDepth) : load_block(rhs_next, sp + kDepth - SP);
      __builtin_amdgcn_sched_barrier(0);
    }
    rhs_cur = rhs_next;
    rhs_next = window_ptr(c0 + 2 * c_step);
    if constexpr (kPerWave) {
      // (the stores below are divergent and the block's only consumer)
      keep_result_in_all_lanes(acc);
      constexpr bool rows_out = kRows;
      const int j = rotated(c0 >> 5);      // (whole outer columns in this form)
      store_t* tile = (store_t*)a.out + (rows_out ? (int64_t)j * 32 : (int64_t)j * a.out_stride_elems);
      // Register v of lane l is row l % 32, column 8 (v / 4) + 4 (l / 32) + v % 4:
      // stored from there, the M0 x 32 sums of a narrow tile are 16 store
      // instructions with 2 M0 lanes each, and a compute unit takes a memory
      // instruction only every 30-50 cycles whatever it moves: with M0 = 1 the
      // stores of this form cost twice what its 8 loads per outer column do.
      // The wave passes the block through its own part of LDS instead (no
      // barrier: a wave's LDS accesses are served in order) and stores element
      // e = 64 i + lane of the tile from lane `lane`: M0 / 2 instructions.
      sum_t (*mine)[64] = partial[0][wave];
#pragma unroll
      for (int v = 0; v < 16; ++v) mine[v][lane] = acc[v];
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      const int elems = a.M0 * 32;
#pragma unroll 1
      for (int e = lane; e < elems; e += 64) {
        // (tiles stored transposed hold element (mm, nn) at nn * M0 + mm)
        const int mm = a.transpose_out ? e % a.M0 : e >> 5, nn = a.transpose_out ? e / a.M0 : e & 31;
        if (rows_out && j * 32 + nn >= a.out_cols) continue;
        const int v = ((nn >> 3) << 2) | (nn & 3), l = mm + 32 * ((nn >> 2) & 1);
        const int64_t at = rows_out ? mm * a.out_row_pitch_elems + nn : e;
        const sum_t sum = (a.accumulate ? (sum_t)tile[at] : (sum_t)0) + mine[v][l];
        tile[at] = (store_t)sum;
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      continue;
    }
    // ---- sum the 8 K slices in wave order and store -----------------------
    sum_t (*buf)[16][64] = partial[parity];
#pragma unroll
    for (int v = 0; v < 16; ++v) buf[wave][v][lane] = acc[v];
    __syncthreads();
    constexpr bool rows_out = kRows;
    store_t* const out_row = (store_t*)a.out + blockIdx.y * a.chunk_out_elems;
#pragma unroll
    for (int rep = 0; rep < 2; ++rep) {
      const int flat = rep * kThreads + threadIdx.x;   // v * 64 + lane
      const int l = flat & 63, v = flat >> 6;
      const int mm = l & 31;
      const int c = c0 + 8 * (v >> 2) + 4 * (l >> 5) + (v & 3);       // this sum's column
      const int nn = c & 31;                                          // ... inside its outer column
      if (mm < a.M0 && c < c_lim && !(rows_out && c >= a.out_cols)) {
        store_t* tile = out_row + (rows_out ? (int64_t)(c - nn) : (int64_t)(c >> 5) * a.out_stride_elems);
        const int64_t at = rows_out ? mm * a.out_row_pitch_elems + nn
                                    : a.transpose_out ? nn * a.M0 + mm : mm * 32 + nn;
        sum_t sum = a.accumulate ? (sum_t)tile[at] : (sum_t)0;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) sum += buf[w][v][l];
        tile[at] = (store_t)sum;
      }
    }
    // The other half of `partial` serves the next tile; this half is rewritten
    // two tiles later, after the next tile's barrier.
  }
}

// chunks: workgroup rows, each taking a.chunk_steps K steps; with more than one
// the results are partial sums in the accumulator's type.
// One launch of the form that splits K over the waves, with the left-hand side
// staged through LDS when the slices of the 8 waves fit 64 KiB of it (narrow
// tiles of up to 8 rows at the longest K a launch takes).
template <typename Cfg, int SP, bool kPartialOut, bool kRows = false, bool kTail = false>
int launch_split_form(SkinnyArgs a, dim3 grid, hipStream_t s) {
  if constexpr (!kRows && !kTail) {
    if (a.tail_tiles) return launch_split_form<Cfg, SP, kPartialOut, false, true>(a, grid, s);
  }
  void (*kernel)(SkinnyArgs) = mmt4d_skinny_kernel<Cfg, SP, kPartialOut, false, kRows, kTail>;
  constexpr bool rows_lhs = kRows;
  const int step_bytes = rows_lhs ? 32 * Cfg::kSub : (Cfg::kSub == 2 ? 4 : a.half_k0 ? 2 : 1) * a.lhs_tile_bytes;
  // (row-major: M0 rows of SP steps and 16 bytes, and room for the last load of the last row)
  const int wave_bytes = rows_lhs ? (a.M0 * (SP * step_bytes + 16) + 1024 + 1023) / 1024 * 1024
                                  : (SP * step_bytes + 1023) / 1024 * 1024;
  size_t lds = 0;
  a.stage_wave_bytes = 0;
  // (the kernel's static partial sums take 64 KiB of the 160)
  constexpr int kMaxStageBytes = 96 * 1024;
  if (kWaves * wave_bytes <= (rows_lhs ? kMaxStageBytes : 64 * 1024)) {
    a.stage_wave_bytes = wave_bytes;
    lds = (size_t)kWaves * wave_bytes;
    // (with the kernel's static partial sums this is more than the default 64 KiB)
    static PerDeviceOnce attr_set_on;
    int dev = 0;
    UK_RETURN_IF_HIP(hipGetDevice(&dev));
    if (!attr_set_on.done(dev)) {
      UK_RETURN_IF_HIP(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kMaxStageBytes));
      attr_set_on.mark(dev);
    }
  }
  hipLaunchKernelGGL(kernel, grid, dim3(kThreads), lds, s, a);
  return check_hip(hipGetLastError(), "mmt4d_skinny launch");
}

template <typename Cfg, bool kRows = false>
int launch_cfg(SkinnyArgs a, int chunks, hipStream_t s) {
  const int cus = device_cu_count();
  // (a batch: about two workgroups per compute unit over all planes)
  int per_plane = a.batch > 1 ? (2 * cus + a.batch - 1) / a.batch : cus;
  per_plane = per_plane > cus ? cus : per_plane;
  constexpr bool kNarrowOut = sizeof(typename Cfg::out_t) < 4;
  // (fp8: up to 8 steps; 16 of its 8-register fragments would not fit beside
  // the rolling buffer)
  constexpr int kPerWaveSteps = Cfg::kSub == 2 ? 8 : 16;
  const int groups = (a.N + kWaves - 1) / kWaves;
  if (chunks == 1 && a.chunk_steps <= kPerWaveSteps &&
      (int64_t)groups * (a.batch > 1 ? a.batch : 1) >= cus) {
    // a short K and enough outer columns to give every compute unit 8 of
    // them: one outer column per wave
    a.steps_per_wave = a.chunk_steps;
    a.stage_wave_bytes = 0;
    // (32 planes of 1024 outer columns, 8 MiB apart: 53.3 -> 51.7 us; other
    // amounts measured 51.3 to 53.9)
    a.rot_tiles = a.batch > 1 ? a.N / a.batch : 0;
    const dim3 grid(groups < per_plane ? groups : per_plane, 1, a.batch > 1 ? a.batch : 1);
    void (*kernel)(SkinnyArgs) = nullptr;
    if (a.chunk_steps <= 8) {
      kernel = mmt4d_skinny_kernel<Cfg, 8, false, true, kRows>;
      if constexpr (!kRows) {
        if (a.tail_tiles) kernel = mmt4d_skinny_kernel<Cfg, 8, false, true, false, true>;
      }
    } else if constexpr (kPerWaveSteps >= 16) {
      kernel = mmt4d_skinny_kernel<Cfg, 16, false, true, kRows>;
      if constexpr (!kRows) {
        if (a.tail_tiles) kernel = mmt4d_skinny_kernel<Cfg, 16, false, true, false, true>;
      }
    }
    if (!kernel) return IREE_AMD_UK_STATUS_NOT_FOUND;
    hipLaunchKernelGGL(kernel, grid, dim3(kThreads), 0, s, a);
    return check_hip(hipGetLastError(), "mmt4d_skinny launch");
  }
  // (one workgroup per compute unit walking its tiles: giving every tile a
  // workgroup of its own, two resident per compute unit, so that 448 tiles on
  // 256 compute units all stream at once, measured 24.0 against 22.8 us)
  // Workgroups of a launch row: one per compute unit at most, and at least 16
  // columns each (fewer outer columns than compute units are dealt out in
  // halves: N = 4096, K = 4096 f16 as 256 workgroups of 16 columns 8.4 us, as
  // 128 of 32 with K split over two rows and the launch that adds them 10.85;
  // K = 1024: 4.8 against 7.4).
  int blocks = a.N < per_plane ? a.N : per_plane;
  if (a.batch <= 1) blocks = a.N * 2 < per_plane ? a.N * 2 : per_plane;
  // K split over workgroup rows: the rows share the compute units, one round in
  // all, each workgroup walking more columns (N = 4096, K = 14336 f16 at 8 rows:
  // 4 rows of 128 workgroups, two rounds, 27.8 us; 4 rows of 64: 25.65; N = 8192,
  // K = 7168: 27.3 -> 24.5).
  if (chunks > 1 && a.batch <= 1) {
    int share = cus / chunks;
    share = share < 1 ? 1 : share;
    blocks = blocks < share ? blocks : share;
  }
  const int per = (a.chunk_steps + kWaves - 1) / kWaves;
  a.steps_per_wave = per;
  const dim3 grid(blocks, chunks, a.batch > 1 ? a.batch : 1);
  if (chunks > 1 && kNarrowOut) {
    if constexpr (kNarrowOut) {
      if (per <= 8) return launch_split_form<Cfg, 8, true, kRows>(a, grid, s);
      if (per <= 16) return launch_split_form<Cfg, 16, true, kRows>(a, grid, s);
      if (per <= 32) return launch_split_form<Cfg, 32, true, kRows>(a, grid, s);
    }
    return IREE_AMD_UK_STATUS_NOT_FOUND;
  }
  if (per <= 8) return launch_split_form<Cfg, 8, false, kRows>(a, grid, s);
  if (per <= 16) return launch_split_form<Cfg, 16, false, kRows>(a, grid, s);
  if (per <= 32) {
    // (32 fp8 steps of 8 registers each would not fit the register file)
    if constexpr (Cfg::kSub == 2) return IREE_AMD_UK_STATUS_NOT_FOUND;
    else return launch_split_form<Cfg, 32, false, kRows>(a, grid, s);
  }
  return IREE_AMD_UK_STATUS_NOT_FOUND;
}

int mfma_k_of(uint32_t flags) {
  switch (flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK) {
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F32:
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16F32: return 16;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F16:
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16BF16:
      // one final rounding of an f32 sum: the reference's arithmetic only
      // when intermediate roundings are skipped
      return (flags & IREE_AMD_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS) ? 16 : 0;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F32F32F32: return 8;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32: return 32;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F8E4M3F8E4M3F32: return 64;
    default: return 0;
  }
}

}  // namespace

// Narrow tiles served: M0 < 32 with N0 = 32, or N0 < 32 with M0 = 32 (run with
// the operands exchanged); K0 = half or all of the MFMA's K extent.
bool mmt4d_skinny_supported(uint32_t flags, int M0, int N0, int K0) {
  const int mk = mfma_k_of(flags);
  const bool narrow = (M0 >= 1 && M0 < 32 && N0 == 32) || (N0 >= 1 && N0 < 32 && M0 == 32);
  if (mk == 64) return narrow && K0 == 16;
  return mk && narrow && (K0 == mk || K0 * 2 == mk);
}

namespace {
// MFMA steps one launch can take: the left-hand side of a wave's K slice stays
// in registers (32 steps per wave; 16 for fp8, whose step is twice as large).
int max_steps_per_launch(int mfma_k) { return kWaves * (mfma_k == 64 ? 16 : 32); }

// One launch over the K of `p`: `chunks` workgroup rows of `chunk_steps` K steps
// each; with more than one, the results are partial sums written to `scratch`.
struct BatchStrides { int64_t batch, lhs, rhs, out; };   // strides in elements
int launch_chunk(const iree_amd_uk_mmt4d_params_t& p, int chunks, int chunk_steps, void* scratch,
                 hipStream_t s, const BatchStrides* batch = nullptr);

// The narrow right-hand side form as the narrow left-hand side problem the
// kernel solves: operands exchanged, the 32 x N0 result tiles (one per outer
// row, out_stride0 apart) written transposed. The marker travels in a flag
// bit that no public flag uses.
constexpr uint32_t kTransposedOut = 0x80000000u;
bool narrow_rhs_form(const iree_amd_uk_mmt4d_params_t& p) { return p.N0 < 32 && p.M0 == 32; }
iree_amd_uk_mmt4d_params_t exchanged(const iree_amd_uk_mmt4d_params_t& p) {
  iree_amd_uk_mmt4d_params_t q = p;
  q.lhs_buffer = p.rhs_buffer; q.lhs_offset = p.rhs_offset; q.lhs_stride0 = p.rhs_stride0;
  q.rhs_buffer = p.lhs_buffer; q.rhs_offset = p.lhs_offset; q.rhs_stride0 = p.lhs_stride0;
  q.M = p.N; q.N = p.M;
  q.M0 = p.N0; q.N0 = p.M0;
  q.flags = p.flags | kTransposedOut;
  return q;
}
}  // namespace

// `batch` problems of one narrow shape as the planes of one launch; only what a
// single launch row takes (K short enough to stay in registers), at most 65535
// entries and batch strides of whole 16 bytes.
int launch_batch_mmt4d_skinny(const iree_amd_uk_mmt4d_params_t& p0, int64_t batch, int64_t lhs_batch_stride,
                              int64_t rhs_batch_stride, int64_t out_batch_stride, hipStream_t s) {
  if (!mmt4d_skinny_supported(p0.flags, p0.M0, p0.N0, p0.K0)) return IREE_AMD_UK_STATUS_NOT_FOUND;
  iree_amd_uk_mmt4d_params_t p = p0;
  if (narrow_rhs_form(p0)) {
    p = exchanged(p0);
    const int64_t t = lhs_batch_stride;
    lhs_batch_stride = rhs_batch_stride;
    rhs_batch_stride = t;
  }
  const int mk = mfma_k_of(p.flags);
  const int64_t k_elems = p.K * p.K0;
  // (the kernel counts columns, 32 per outer column, in 32 bits)
  if (p.M != 1 || p.K == 0 || p.N > 0x3FFFFFF || batch > 65535)
    return IREE_AMD_UK_STATUS_NOT_FOUND;
  const int64_t steps = (k_elems + mk - 1) / mk;   // (the last one may be partial)
  if (steps > max_steps_per_launch(mk)) return IREE_AMD_UK_STATUS_NOT_FOUND;
  const BatchStrides bs = {batch, lhs_batch_stride, rhs_batch_stride, out_batch_stride};
  return launch_chunk(p, 1, (int)steps, nullptr, s, &bs);
}

int launch_mmt4d_skinny(const iree_amd_uk_mmt4d_params_t& p0, hipStream_t s) {
  if (!mmt4d_skinny_supported(p0.flags, p0.M0, p0.N0, p0.K0)) return IREE_AMD_UK_STATUS_NOT_FOUND;
  const iree_amd_uk_mmt4d_params_t p = narrow_rhs_form(p0) ? exchanged(p0) : p0;
  const bool transposed = (p.flags & kTransposedOut) != 0;
  const int mk = mfma_k_of(p.flags);
  const int64_t k_elems = p.K * p.K0;
  if (p.M != 1 || p.K == 0 || p.N > 0x3FFFFFF) return IREE_AMD_UK_STATUS_NOT_FOUND;
  // (a K that is not whole steps ends in a partial one)
  const int64_t steps = (k_elems + mk - 1) / mk;
  if (steps > 0x7FFFFFFF) return IREE_AMD_UK_STATUS_NOT_FOUND;
  const int max_steps = max_steps_per_launch(mk);
  Mmt4dTypeInfo ti;
  mmt4d_type_info(p.flags, &ti);
  // K is split over workgroup rows when one launch row cannot hold it in
  // registers, and when the outer columns alone leave half of the compute units
  // or more idle: every row writes its sums (in the accumulator's type) to the
  // stream's scratch buffer, and a second kernel adds them in row order, after
  // the old result when accumulating. Deterministic; exact for integers, for
  // floats the same sum in another order.
  const int cus = device_cu_count();
  int64_t chunks = (steps + max_steps - 1) / max_steps;
  // (partial sums and result are dense arrays there: transposed tiles must
  // follow each other without gaps)
  const bool dense_out = !transposed || p.N == 1 || p.out_stride0 == (int64_t)p.M0 * 32;
  // (column blocks of a launch row: see launch_cfg)
  const int64_t col_blocks = p.N * 2 < cus ? p.N * 2 : cus;
  if (dense_out && col_blocks * chunks * 2 <= cus && steps >= 64) {
    int64_t more = cus / col_blocks;
    if (more > steps / 32) more = steps / 32;
    if (more > 8) more = 8;
    if (more > chunks) chunks = more;
  }
  if (chunks > 1 && dense_out) {
    const int64_t chunk_steps = (steps + chunks - 1) / chunks;
    chunks = (steps + chunk_steps - 1) / chunk_steps;
    const int64_t elems = p.N * p.M0 * 32;
    // (the tiles of the single outer row are consecutive: partial sums and
    // result are dense arrays)
    ScratchLease lease(s, (size_t)(chunks * elems * 4));
    if (lease.overflowed()) return scratch_overflow_status("mmt4d: the K split of a narrow tile", (size_t)(chunks * elems * 4));
    void* scratch = lease.ptr();
    if (scratch && chunks > 1) {
      int st = launch_chunk(p, (int)chunks, (int)chunk_steps, scratch, s);
      if (st) return st;
      KSplitReduceArgs r;
      r.partials = scratch;
      r.slices = (int)chunks;
      r.M = 1; r.N = 1;
      r.flat_elems = elems;
      r.out = (char*)p.out_buffer + p.out_offset * ti.out_bytes;
      r.out_stride_bytes = 0;
      r.accumulate = (p.flags & IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE) != 0;
      r.row_major_out = 0; r.out_rows = r.out_cols = 0;
      r.out_scale = 1.0f;
      r.acc_is_float = (p.flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK) != IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32;
      const uint32_t type = p.flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK;
      r.out_kind = type == IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F16 ? 1
                   : type == IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16BF16 ? 2 : 0;
      return launch_ksplit_reduce(r, s);
    }
  }
  if (steps <= max_steps) return launch_chunk(p, 1, (int)steps, nullptr, s);
  // Without scratch memory a longer K runs as several launches over equal K
  // slices, each accumulating into the result of the one before. Results
  // narrower than the accumulator (f16, bf16) would be rounded between the
  // slices, so those are refused.
  if (ti.out_bytes != 4) return IREE_AMD_UK_STATUS_NOT_FOUND;
  const int64_t n_chunks = (steps + max_steps - 1) / max_steps;
  const int64_t chunk_steps = (steps + n_chunks - 1) / n_chunks;
  const int64_t tiles_per_step_num = mk, tiles_per_step_den = p.K0;   // K tiles per step = mk / K0 (1 or 2; fp8 4)
  for (int64_t first = 0; first < steps; first += chunk_steps) {
    const int64_t n = steps - first < chunk_steps ? steps - first : chunk_steps;
    iree_amd_uk_mmt4d_params_t q = p;
    const int64_t tile0 = first * tiles_per_step_num / tiles_per_step_den;
    q.K = n * tiles_per_step_num / tiles_per_step_den;
    if (q.K > p.K - tile0) q.K = p.K - tile0;     // (the last slice ends with K)
    q.lhs_offset += tile0 * p.M0 * p.K0;
    q.rhs_offset += tile0 * p.N0 * p.K0;
    if (first > 0) q.flags |= IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE;
    const int st = launch_chunk(q, 1, (int)n, nullptr, s);
    // (only the first slice can be refused: alignment and strides are the same for all)
    if (st) return st;
  }
  return 0;
}

namespace {
int launch_chunk(const iree_amd_uk_mmt4d_params_t& p, int chunks, int chunk_steps, void* scratch,
                 hipStream_t s, const BatchStrides* batch) {
  const int mk = mfma_k_of(p.flags);
  Mmt4dTypeInfo ti;
  mmt4d_type_info(p.flags, &ti);
  const int eb = ti.lhs_bits / 8;
  const int64_t k_elems = p.K * p.K0;
  // 16-byte aligned operands
  if (p.N > 0x3FFFFFF) return IREE_AMD_UK_STATUS_NOT_FOUND;
  const char* lhs = (const char*)p.lhs_buffer + p.lhs_offset * eb;
  const char* rhs = (const char*)p.rhs_buffer + p.rhs_offset * eb;
  if (((uintptr_t)lhs | (uintptr_t)rhs) % 16 || (p.rhs_stride0 * eb) % 16 || (p.M0 * p.K0 * eb) % 16)
    return IREE_AMD_UK_STATUS_NOT_FOUND;
  SkinnyArgs a;
  a.rot_tiles = 0;
  a.lhs = lhs; a.rhs = rhs;
  a.out = (char*)p.out_buffer + p.out_offset * ti.out_bytes;
  a.rhs_stride_bytes = p.rhs_stride0 * eb;
  // consecutive outer columns of the single outer row; exchanged operands: the
  // tiles of the caller's outer rows, out_stride0 apart
  a.transpose_out = (p.flags & kTransposedOut) != 0;
  a.out_stride_elems = a.transpose_out ? p.out_stride0 : (int64_t)p.M0 * 32;
  a.N = (int)p.N; a.M0 = p.M0;
  a.ksteps = (int)((k_elems + mk - 1) / mk);
  a.tail_tiles = (int)((k_elems % mk) / p.K0);
  a.steps_per_wave = 0;
  a.lhs_tile_bytes = p.M0 * p.K0 * eb;
  a.half_k0 = p.K0 * 2 == mk;
  a.accumulate = (p.flags & IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE) != 0;
  a.chunk_steps = chunk_steps;
  a.chunk_out_elems = 0;
  a.lhs_row_pitch_bytes = 0;
  a.out_row_pitch_elems = 0;
  a.out_cols = 0;
  a.batch = 1;
  a.lhs_batch_bytes = a.rhs_batch_bytes = a.out_batch_bytes = 0;
  if (batch) {
    a.batch = (int)batch->batch;
    a.lhs_batch_bytes = batch->lhs * eb;
    a.rhs_batch_bytes = batch->rhs * eb;
    a.out_batch_bytes = batch->out * ti.out_bytes;
    if (a.lhs_batch_bytes % 16 || a.rhs_batch_bytes % 16) return IREE_AMD_UK_STATUS_NOT_FOUND;
  }
  if (chunks > 1) {
    a.out = (char*)scratch;
    a.accumulate = 0;
    a.chunk_out_elems = (int64_t)p.N * p.M0 * 32;
    a.out_stride_elems = (int64_t)p.M0 * 32;     // (partial sums are dense)
  }
  switch (p.flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK) {
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F32: return launch_cfg<F16Cfg>(a, chunks, s);
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16F32: return launch_cfg<BF16Cfg>(a, chunks, s);
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32: return launch_cfg<S8Cfg>(a, chunks, s);
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F32F32F32: return launch_cfg<F32Cfg>(a, chunks, s);
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F8E4M3F8E4M3F32: return launch_cfg<F8Cfg>(a, chunks, s);
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F16: return launch_cfg<F16F16Cfg>(a, chunks, s);
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16BF16: return launch_cfg<BF16BF16Cfg>(a, chunks, s);
    default: return IREE_AMD_UK_STATUS_NOT_FOUND;
  }
}
}  // namespace

// The whole linear layer on a few rows: out[M][out_cols] (+)= lhs[M][K] * rhs,
// lhs and out row-major (`p` describes them as iree_amd_uk_matmul_packed_rhs
// does: lhs_stride0 and out_stride0 are row pitches in elements), rhs packed
// 32 x K0 tiles, 1 < M <= 32. One launch of the kernel above with the rows of
// the matrix as the rows of its single narrow tile; NOT_FOUND for what that
// launch cannot take (a K that one launch row cannot hold in registers, too
// few outer columns to be worth it, operands that are not 16-byte aligned).
int launch_matmul_rows_skinny(const iree_amd_uk_mmt4d_params_t& p, int64_t M, int64_t out_cols, hipStream_t s) {
  if (M < 2 || M > 32 || !mmt4d_skinny_supported(p.flags, 16, 32, p.K0)) return IREE_AMD_UK_STATUS_NOT_FOUND;
  const int mk = mfma_k_of(p.flags);
  Mmt4dTypeInfo ti;
  mmt4d_type_info(p.flags, &ti);
  const int eb = ti.lhs_bits / 8;
  const int64_t k_elems = p.K * p.K0;
  if (p.K == 0 || k_elems % mk || p.N > 0x3FFFFFF || out_cols > 0x7FFFFFFF) return IREE_AMD_UK_STATUS_NOT_FOUND;
  // (measured at N = 14336, K = 4096: 2-byte elements at 31 / 32 rows 29.0 /
  // 29.7 us against 28.4 for the macro-tile kernel, 26.9 at 24 rows; 1-byte
  // elements at 32 rows 15.1 (i8) and 16.7 (fp8) against 17.2 and 17.0)
  if (eb > 1 && M > 24) return IREE_AMD_UK_STATUS_NOT_FOUND;
  const int64_t steps = k_elems / mk;
  // (a K longer than one launch row keeps in registers goes to the macro-tile
  // kernel with its K split, which measures as fast or faster there)
  if (steps > max_steps_per_launch(mk)) return IREE_AMD_UK_STATUS_NOT_FOUND;
  // Few outer columns: K is split over workgroup rows as in launch_mmt4d_skinny,
  // every row writing row-major f32 (s32) sums to the stream's scratch buffer,
  // which the reduction kernel adds in row order into a result without gaps
  // between its rows.
  const int cus = device_cu_count();
  int64_t chunks = 1;
  if (p.N * 2 <= cus && steps >= 64) {
    chunks = cus / p.N;
    if (chunks > steps / 32) chunks = steps / 32;
    if (chunks > 8) chunks = 8;
    if (chunks < 1) chunks = 1;
  }
  if (p.N * 2 <= cus && chunks < 2) return IREE_AMD_UK_STATUS_NOT_FOUND;
  if (chunks > 1 && (p.out_stride0 != out_cols || (M * out_cols) % 4)) return IREE_AMD_UK_STATUS_NOT_FOUND;
  const char* lhs = (const char*)p.lhs_buffer + p.lhs_offset * eb;
  const char* rhs = (const char*)p.rhs_buffer + p.rhs_offset * eb;
  if (((uintptr_t)lhs | (uintptr_t)rhs) % 16 || (p.rhs_stride0 * eb) % 16 || (p.lhs_stride0 * eb) % 16)
    return IREE_AMD_UK_STATUS_NOT_FOUND;
  if (M * p.lhs_stride0 * eb > 0x7FFFFFFF) return IREE_AMD_UK_STATUS_NOT_FOUND;
  SkinnyArgs a;
  a.rot_tiles = 0;
  a.lhs = lhs; a.rhs = rhs;
  a.out = (char*)p.out_buffer + p.out_offset * ti.out_bytes;
  a.rhs_stride_bytes = p.rhs_stride0 * eb;
  a.transpose_out = 0;
  a.out_stride_elems = 0;
  a.N = (int)p.N; a.M0 = (int)M;
  a.ksteps = (int)steps;
  a.tail_tiles = 0;
  a.steps_per_wave = 0;
  a.lhs_tile_bytes = 0;
  a.half_k0 = p.K0 * 2 == mk;
  a.accumulate = (p.flags & IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE) != 0;
  a.chunk_steps = (int)steps;
  a.chunk_out_elems = 0;
  a.lhs_row_pitch_bytes = p.lhs_stride0 * eb;
  a.out_row_pitch_elems = p.out_stride0;
  a.out_cols = (int)out_cols;
  a.batch = 1;
  a.lhs_batch_bytes = a.rhs_batch_bytes = a.out_batch_bytes = 0;
  std::unique_ptr<ScratchLease> lease;   // held until the reduction has been queued
  if (chunks > 1) {
    const int64_t chunk_steps = (steps + chunks - 1) / chunks;
    chunks = (steps + chunk_steps - 1) / chunk_steps;
    if (chunks < 2) return IREE_AMD_UK_STATUS_NOT_FOUND;
    lease.reset(new ScratchLease(s, (size_t)(chunks * M * out_cols * 4)));
    if (!lease->ptr()) return IREE_AMD_UK_STATUS_NOT_FOUND;
    a.out = (char*)lease->ptr();
    a.accumulate = 0;
    a.chunk_steps = (int)chunk_steps;
    a.chunk_out_elems = M * out_cols;
    a.out_row_pitch_elems = out_cols;
  }
  int st;
  switch (p.flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK) {
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F32: st = launch_cfg<F16Cfg, true>(a, (int)chunks, s); break;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16F32: st = launch_cfg<BF16Cfg, true>(a, (int)chunks, s); break;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32: st = launch_cfg<S8Cfg, true>(a, (int)chunks, s); break;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F32F32F32: st = launch_cfg<F32Cfg, true>(a, (int)chunks, s); break;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F8E4M3F8E4M3F32: st = launch_cfg<F8Cfg, true>(a, (int)chunks, s); break;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F16: st = launch_cfg<F16F16Cfg, true>(a, (int)chunks, s); break;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16BF16: st = launch_cfg<BF16BF16Cfg, true>(a, (int)chunks, s); break;
    default: return IREE_AMD_UK_STATUS_NOT_FOUND;
  }
  if (st || chunks == 1) return st;
  KSplitReduceArgs r;
  r.partials = lease->ptr();
  r.slices = (int)chunks;
  r.M = 1; r.N = 1;
  r.flat_elems = M * out_cols;
  r.out = (char*)p.out_buffer + p.out_offset * ti.out_bytes;
  r.out_stride_bytes = 0;
  r.accumulate = (p.flags & IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE) != 0;
  r.row_major_out = 0; r.out_rows = r.out_cols = 0;
  r.out_scale = 1.0f;
  r.acc_is_float = (p.flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK) != IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32;
  const uint32_t type = p.flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK;
  r.out_kind = type == IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F16 ? 1
               : type == IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16BF16 ? 2 : 0;
  return launch_ksplit_reduce(r, s);
}

}  // namespace uk
