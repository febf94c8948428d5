// Launch side of the matrix-core mmt4d kernels: the __global__ wrapper, the
// choice of the macro tile for a problem, the split of a partial last round
// and the split of K for problems of few macro tiles.
// Included by the translation units that instantiate the kernels of one
// element-type tuple each (uk_mmt4d_mfma_inst_*.hip), so that they compile in
// parallel; uk_mmt4d_mfma.hip calls them through the functions declared here.
#ifndef IREE_AMD_UK_MMT4D_MFMA_LAUNCH_H_
#define IREE_AMD_UK_MMT4D_MFMA_LAUNCH_H_

#include "uk_common.h"
#include "uk_mmt4d_mfma_kernel.h"

namespace uk {

// One per element-type tuple (f16 / bf16 on the 16-row instruction shapes).
int launch_mfma_f16f16f32(const MfmaArgs& a, hipStream_t s);
int launch_mfma_f16f16f16(const MfmaArgs& a, hipStream_t s);
int launch_mfma_bf16bf16f32(const MfmaArgs& a, hipStream_t s);
int launch_mfma_bf16bf16bf16(const MfmaArgs& a, hipStream_t s);
int launch_mfma_s8s8s32(const MfmaArgs& a, hipStream_t s);
int launch_mfma_f32f32f32(const MfmaArgs& a, hipStream_t s);
int launch_mfma_f8f8f32(const MfmaArgs& a, hipStream_t s);
// With the fused SiLU * up epilogue (e4m3 result).
int launch_mfma_silu_f16(const MfmaArgs& a, hipStream_t s);
int launch_mfma_silu_bf16(const MfmaArgs& a, hipStream_t s);
int launch_mfma_silu_f8(const MfmaArgs& a, hipStream_t s);

namespace {

// kOcc: waves per SIMD the register allocation must leave room for (2 = two
// workgroups of 4 waves resident on one compute unit).
template <typename Cfg, int WM, int WN, int kRing, int kSync, int kOcc, bool kSiluMul, int kWavesN,
          int kForm>
__global__ __launch_bounds__(128 * kWavesN, kOcc) void mmt4d_mfma_kernel(MfmaArgs a) {
  // Plane blockIdx.z of a batch (the strides are 0 without one). Workgroups go
  // to the 8 XCDs round-robin in launch order, which deals the few macro tiles
  // of a small batch entry over all XCDs: no two tiles of a row share an L2
  // and every tile fetches its operands from memory by itself (32 x 512^3 f16:
  // 22.9 us; 16.2 with whole entries per XCD). So the first batch_by_xcd planes
  // (a multiple of 8, set for entries of at most 64 tiles) are dealt whole:
  // workgroup L of the launch takes tile (L / 8) % tiles of plane
  // L % 8 + 8 * (L / 8 / tiles); the planes after them stay as launched.
  unsigned plane = blockIdx.z, bid = blockIdx.x;
  if (blockIdx.z < (unsigned)a.batch_by_xcd) {
    const unsigned linear = blockIdx.z * gridDim.x + blockIdx.x;
    const unsigned j = linear / 8;
    plane = linear % 8 + 8 * (j / gridDim.x);
    bid = j % gridDim.x;
  }
  a.lhs += plane * a.lhs_batch_bytes;
  a.rhs += plane * a.rhs_batch_bytes;
  a.out += plane * a.out_batch_bytes;
  mmt4d_mfma_body<Cfg, WM, WN, kRing, kSync, kSiluMul, kWavesN, kForm>(a, (int)bid);
}

// K split: workgroup row blockIdx.y multiplies its slice of K into its own
// tiled partial result.
template <typename Cfg, int WM, int WN, int kRing, int kSync, int kOcc, int kWavesN, int kForm>
__global__ __launch_bounds__(128 * kWavesN, kOcc) void mmt4d_mfma_ksplit_kernel(MfmaArgs a) {
  static_assert(kForm == 0 || kForm == 3, "partial results are tiled");
  // bytes of one K-step in an outer row of packed tiles / in a row of a row-major matrix
  constexpr int64_t kPackedStep = (32 / Cfg::kRows) * Cfg::kSub * 1024;
  constexpr int64_t kRowStep = (64 / Cfg::kRows) * 16 * Cfg::kSub;
  const int slice = blockIdx.y;
  const int first = slice * a.slice_ksteps;
  a.lhs += first * (kForm == 3 ? kRowStep : kPackedStep);
  a.rhs += first * kPackedStep;
  a.out += slice * a.slice_out_bytes;
  if (slice == a.k_slices - 1) {
    a.ksteps -= first;
  } else {
    a.ksteps = a.slice_ksteps;
    a.tail_tiles = 0;
  }
  mmt4d_mfma_body<Cfg, WM, WN, kRing, kSync, false, kWavesN, kForm, false>(a);
}

template <typename Cfg, int WM, int WN, int kRing, int kSync, int kOcc, bool kSiluMul, int kWavesN,
          int kForm>
int launch_form(const MfmaArgs& a, unsigned blocks, hipStream_t s) {
  constexpr int lds_bytes = mmt4d_mfma_lds_bytes<Cfg, WM, WN, kRing, kWavesN>();
  static_assert(lds_bytes <= 160 * 1024, "LDS ring exceeds 160 KiB");
  // (form 3 exists only as the K-split kernel, and partial sums only in the
  // accumulator type)
  constexpr bool kCanSplit = !kSiluMul && (kForm == 0 || kForm == 3) &&
                             std::is_same<typename PartialSumCfg<Cfg>::type, Cfg>::value;
  void (*kernel)(MfmaArgs) = nullptr;
  unsigned slices = 1;
  if (a.k_slices > 1) {
    if (a.batch > 1) return IREE_AMD_UK_STATUS_NOT_FOUND;
    if constexpr (kCanSplit) {
      kernel = mmt4d_mfma_ksplit_kernel<Cfg, WM, WN, kRing, kSync, kOcc, kWavesN, kForm>;
      slices = (unsigned)a.k_slices;
    }
  } else {
    if constexpr (kForm != 3) kernel = mmt4d_mfma_kernel<Cfg, WM, WN, kRing, kSync, kOcc, kSiluMul, kWavesN, kForm>;
  }
  if (!kernel) return IREE_AMD_UK_STATUS_NOT_FOUND;
  // The attribute belongs to the kernel on ONE device: set it once per device
  // ordinal.
  static PerDeviceOnce attr_set_on[2];
  PerDeviceOnce& set_on = attr_set_on[slices > 1];
  int dev = 0;
  UK_RETURN_IF_HIP(hipGetDevice(&dev));
  if (!set_on.done(dev)) {
    UK_RETURN_IF_HIP(hipFuncSetAttribute((const void*)kernel,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes));
    set_on.mark(dev);
  }
  MfmaArgs b = a;
  b.batch_by_xcd = a.batch >= 8 && blocks <= 64 ? a.batch / 8 * 8 : 0;
  hipLaunchKernelGGL(kernel, dim3(blocks, slices, a.batch > 1 ? (unsigned)a.batch : 1u), dim3(128 * kWavesN),
                     lds_bytes, s, b);
  return check_hip(hipGetLastError(), "mmt4d_mfma launch");
}

template <typename Cfg, int WM, int WN, int kRing, int kSync, int kOcc = 1, bool kSiluMul = false,
          int kWavesN = 2>
int launch_variant(const MfmaArgs& a0, hipStream_t s) {
  MfmaArgs a = a0;
  constexpr int kPerTile = 32 / Cfg::kRows;
  constexpr int TM = 2 * WM, TN = kWavesN * WN;   // blocks of Cfg::kRows rows
  static_assert(TM % kPerTile == 0 && TN % kPerTile == 0, "a workgroup covers whole outer tiles");
  // (the fp8 MLP block, whose matmuls run on 128 x 256 tiles: 289-292 us in
  // panels of 4 rows, 286-288 in panels of 8, 309 in panels of 16)
  a.panel_rows = WM < WN ? 8 : 4;
  a.tiles_m = (a.M * kPerTile + TM - 1) / TM;
  a.tiles_n = (a.N * kPerTile + TN - 1) / TN;
  const int64_t blocks = (int64_t)a.tiles_m * a.tiles_n;
  if (blocks > 0x7FFFFFFF) return IREE_AMD_UK_STATUS_NOT_FOUND;
  // one kernel instance per operand form (the forms the entry points produce)
  constexpr bool kPackedLhs = !RowMajorLhsOnly<Cfg>::value;
  if constexpr (!kSiluMul) {
    if (a.k_slices > 1 && a.row_major_out) return IREE_AMD_UK_STATUS_NOT_FOUND;
    if (a.lhs_row_major && a.row_major_out)
      return launch_form<Cfg, WM, WN, kRing, kSync, kOcc, kSiluMul, kWavesN, 2>(a, (unsigned)blocks, s);
    if constexpr (kPackedLhs) {
      if (a.row_major_out)
        return launch_form<Cfg, WM, WN, kRing, kSync, kOcc, kSiluMul, kWavesN, 1>(a, (unsigned)blocks, s);
    }
  }
  if constexpr (!kSiluMul) {
    if (a.lhs_row_major)   // (tiled result: the partial sums of a K split)
      return launch_form<Cfg, WM, WN, kRing, kSync, kOcc, kSiluMul, kWavesN, 3>(a, (unsigned)blocks, s);
  }
  if (a.lhs_row_major || a.row_major_out) return IREE_AMD_UK_STATUS_NOT_FOUND;
  if constexpr (kPackedLhs)
    return launch_form<Cfg, WM, WN, kRing, kSync, kOcc, kSiluMul, kWavesN, 0>(a, (unsigned)blocks, s);
  else
    return IREE_AMD_UK_STATUS_NOT_FOUND;
}

// The four macro tiles (in outer tiles of 32 rows: 8x8, 8x4, 4x8, 4x4) with
// their LDS rings: 8 K-steps and a barrier every 2 for the single-occupancy
// tiles (fp8 and the 16-row shapes, whose K-step is twice as large: 5 and every
// step), 6 (wide: 3) for the double-occupancy ones.
template <typename Cfg, bool kSiluMul>
int launch_by_index(int v, const MfmaArgs& b, hipStream_t s) {
  constexpr int S = 32 / Cfg::kRows;
  constexpr bool kWide = Cfg::kSub == 2 || S == 2;
  switch (v) {
    case 0: return launch_variant<Cfg, 4 * S, 4 * S, kWide ? 5 : 8, kWide ? 1 : 2, 1, kSiluMul>(b, s);
    case 1: return launch_variant<Cfg, 4 * S, 2 * S, kWide ? 3 : 6, kWide ? 1 : 2, 2, kSiluMul>(b, s);
    case 2: return launch_variant<Cfg, 2 * S, 4 * S, kWide ? 3 : 6, kWide ? 1 : 2, 2, kSiluMul>(b, s);
    default: return launch_variant<Cfg, 2 * S, 2 * S, S == 2 ? 4 : 8, S == 2 ? 1 : 2, 1, kSiluMul>(b, s);
  }
}

// K split: `slices` workgroup rows multiply one slice of K each into tiled
// partial results in the stream's scratch buffer, which a second kernel
// sums in slice order into the result (deterministic; integer results are
// those of the unsplit kernel, float results differ from it in the order of
// the additions only). Returns NOT_FOUND when the scratch memory cannot be had
// (the caller then runs unsplit).
template <typename Cfg>
int launch_k_split(const MfmaArgs& a, int v, int slices, hipStream_t s) {
  typedef typename PartialSumCfg<Cfg>::type PCfg;
  typedef typename PCfg::out_t acc_elem_t;
  const int slice_ksteps = (a.ksteps + slices - 1) / slices;
  slices = (a.ksteps + slice_ksteps - 1) / slice_ksteps;      // (no empty last slice)
  if (slices < 2) return IREE_AMD_UK_STATUS_NOT_FOUND;
  const int64_t slice_bytes = (int64_t)a.M * a.N * 1024 * (int64_t)sizeof(acc_elem_t);
  // (held until the reduction kernel has been queued)
  ScratchLease lease(s, (size_t)(slice_bytes * slices));
  if (lease.overflowed()) return scratch_overflow_status("mmt4d: the K split", (size_t)(slice_bytes * slices));
  void* scratch = lease.ptr();
  if (!scratch) return IREE_AMD_UK_STATUS_NOT_FOUND;
  MfmaArgs p = a;
  p.out = (char*)scratch;
  p.out_stride_bytes = (int64_t)a.N * 1024 * (int64_t)sizeof(acc_elem_t);
  p.row_major_out = 0;
  p.accumulate = 0;
  p.out_scale = 1.0f;
  p.k_slices = slices;
  p.slice_ksteps = slice_ksteps;
  p.slice_out_bytes = slice_bytes;
  int st = launch_by_index<PCfg, false>(v, p, s);
  if (!st) {
    KSplitReduceArgs r;
    r.partials = scratch;
    r.slices = slices;
    r.M = a.M; r.N = a.N;
    r.flat_elems = 0;
    r.out = a.out;
    r.out_stride_bytes = a.out_stride_bytes;
    r.accumulate = a.accumulate;
    r.row_major_out = a.row_major_out;
    r.out_rows = a.out_rows; r.out_cols = a.out_cols;
    r.out_scale = a.out_scale;
    r.acc_is_float = std::is_floating_point<acc_elem_t>::value;
    r.out_kind = std::is_same<typename Cfg::out_t, acc_elem_t>::value ? 0
                 : std::is_same<typename Cfg::out_t, _Float16>::value ? 1 : 2;
    st = launch_ksplit_reduce(r, s);
  }
  return st;
}

template <typename Cfg, bool kSiluMul = false>
int launch_cfg(const MfmaArgs& a, hipStream_t s) {
  // Pick the macro tile. 256x256 (one workgroup per compute unit, all of its
  // registers) has the best operand reuse: 1 KiB of operand per two MFMAs.
  // 256x128 / 128x256 run two workgroups per compute unit, so one workgroup's
  // output stores overlap the other's MFMAs, and they spread a problem over
  // more compute units; 128x128 spreads small problems further still.
  // Estimated cost of a variant, in units of one 32x32 block row of MFMAs:
  // rounds of resident workgroups x work per workgroup / relative efficiency
  // (measured on MI355X against the 256x256 tile's rate).
  // LDS rings: 8 K-steps with a barrier every 2 for the single-occupancy
  // tiles (fp8, whose K-step is twice as large: 5 with a barrier every step),
  // 6 (fp8: 3) for the double-occupancy ones.
  const int cus = device_cu_count();
  // (fp8 runs the two-per-compute-unit tiles on a ring of only 3 K-steps:
  // 2048 x 28672 x 4096 measured 238 us with the large tile, 267 with 256x128.
  // With the SiLU epilogue, whose arithmetic the second workgroup hides and
  // whose output is an eighth of the bytes, it is the other way round: 218
  // against 198 us.)
  // S: blocks per 32 rows. The 16-row shapes and fp8 have K-steps of twice the
  // bytes ("wide"), hence the shorter rings.
  constexpr int S = 32 / Cfg::kRows;
  constexpr bool kWide = Cfg::kSub == 2 || S == 2;
  constexpr bool kShallow = Cfg::kSub == 2 && !kSiluMul;
  struct Variant { int wm, wn, occ; double eff_alone, eff_full; };
  // (16-row shapes: 256x128 measured 115 us against 104 for 256x256 at 4096^3)
  constexpr double kEffAlone = kSiluMul ? 1.0 : kShallow ? 0.85 : S == 2 ? 0.86 : 0.9;
  constexpr double kEffFull = kSiluMul ? 1.05 : kShallow ? 0.82 : S == 2 ? 0.9 : 0.94;
  static const Variant variants[4] = {{4, 4, 1, 1.0, 1.0},
                                      {4, 2, 2, kEffAlone, kEffFull},
                                      {2, 4, 2, kEffAlone, kEffFull},
                                      {2, 2, 2, 0.7, 0.75}};
  // cost of variant v on an M x N (outer tiles) problem
  auto cost_of = [&](int v, int64_t M, int64_t N, int64_t k_slices = 1) -> double {
    const Variant& t = variants[v];
    const int64_t tiles = ceil_div(M, (int64_t)2 * t.wm) * ceil_div(N, (int64_t)2 * t.wn) * k_slices *
                          (a.batch > 1 ? a.batch : 1);
    const int64_t slots = (int64_t)t.occ * cus;
    const double work = t.wm * t.wn;
    double cost = (double)(tiles / slots) * t.occ * work / t.eff_full;
    const int64_t rest = tiles % slots;
    if (rest > 0) {
      const int resident = (int)ceil_div(rest, (int64_t)cus);   // workgroups sharing a compute unit
      cost += resident * work / (resident == t.occ ? t.eff_full : t.eff_alone);
    }
    // Of the two half-size tiles the one with more columns than rows is the
    // faster one for the SiLU form (the gate/up matmul of the fp8 MLP block
    // alone, sustained: 187.7 -> 180.0 us; inside the block 292 -> 289). For
    // row-major results on the 32-row instructions the two measure either way:
    // 128x256 ahead by 3-7 % when the call is repeated on operands that stay
    // in the last-level cache (fp8 2048 x 4096 x 14336 100.6 -> 97.4 us),
    // 256x128 ahead by 2 % inside the MLP block, where the weights come from
    // memory every time (block 289 -> 283 us): the latter is what a model does,
    // so those keep the first of the two.
    if (kSiluMul && Cfg::kRows == 32 && v == 1) cost *= 1.03;
    // A row-major left-hand side is the dearer operand to fetch (half or
    // quarter cache lines per row and K-step, each line asked for again on the
    // next step): tiles with more rows than columns pay most. Measured at
    // 2048 x 4096 x 4096 against the packed operand, K-steps of 64 bytes of a
    // row (f16, i8 on the 16-row instruction; fp8 alike): 256x256 1.01,
    // 256x128 1.09-1.14, 128x256 1.02-1.03, 128x128 1.13; K-steps of 32 bytes
    // (i8 otherwise): 1.16, 1.37, 1.06, 1.28.
    if (a.lhs_row_major) {
      constexpr bool kHalfLines = Cfg::kRows == 16 || Cfg::kSub == 2;
      static const double penalty[2][4] = {{1.16, 1.37, 1.06, 1.28}, {1.02, 1.13, 1.03, 1.13}};
      cost *= penalty[kHalfLines][v];
    }
    return cost;
  };
  auto pick = [&](int64_t M, int64_t N, double* out_cost) -> int {
    int best = 0;
    double best_cost = 0;
    for (int v = 0; v < 4; ++v) {
      const double cost = cost_of(v, M, N);
      if (v == 0 || cost < best_cost * 0.999) { best = v; best_cost = cost; }
    }
    *out_cost = best_cost;
    return best;
  };
  auto launch = [&](int v, const MfmaArgs& b) -> int { return launch_by_index<Cfg, kSiluMul>(v, b, s); };
  double best_cost = 0;
  const int best = pick(a.M, a.N, &best_cost);
  // Few macro tiles and a long K (a few hundred rows against a wide K, as in the
  // down projection of an MLP at small batch) leave most compute units idle:
  // K is then split over workgroup rows. Estimated times in microseconds: cost
  // units (block rows of MFMAs per K-step) x K-steps x the measured time of a
  // unit, plus, for a split, the second launch and the traffic of the partial
  // sums (written once, read once, at about 3 TB/s).
  if constexpr (!kSiluMul) {
    const Variant& bv = variants[best];
    const int64_t best_tiles = ceil_div((int64_t)a.M, (int64_t)2 * bv.wm) * ceil_div((int64_t)a.N, (int64_t)2 * bv.wn);
    if (a.k_slices == 0 && a.batch <= 1 && a.ksteps >= 64 && best_tiles * 2 <= (int64_t)bv.occ * cus) {
      const double unit_us = Cfg::kStepUs / 16.0;
      const double out_mb = (double)a.M * a.N * 4096.0 / 1e6;
      // A split must win by 5 % (with 10 %, 512 x 4096 x 4096 f16 stayed unsplit
      // at 31.2 us where two slices of 128x128 tiles take 26.5; over 21 shapes
      // of few tiles in f16 and i8 the lower bar gained up to 15 % and cost at
      // most 4 %).
      double best_us = best_cost * a.ksteps * unit_us * 0.95;
      int split_v = -1, split_n = 0;
      for (int v = 0; v < 4; ++v) {
        // (up to 64 rows: with the tile and slice count forced, 128x128 tiles
        // won on every such shape measured, by up to 10 % over what this
        // estimate picked among the larger tiles, whose rows are as idle and
        // whose workgroups are half as many)
        if (a.M <= 2 && v != 3) continue;
        for (int n = 2; n <= 8; ++n) {
          if (a.ksteps / n < 24) break;
          const int64_t tiles = ceil_div((int64_t)a.M, (int64_t)2 * variants[v].wm) *
                                ceil_div((int64_t)a.N, (int64_t)2 * variants[v].wn) * n;
          if (tiles > (int64_t)variants[v].occ * cus) break;     // at most one round
          const double us = cost_of(v, a.M, a.N, n) * ceil_div((int64_t)a.ksteps, (int64_t)n) * unit_us + 6.0 +
                            (n + 1 + (a.accumulate ? 1 : 0)) * out_mb / 3.0;
          if (us < best_us) { best_us = us; split_v = v; split_n = n; }
        }
      }
      if (split_n > 1) {
        const int st = launch_k_split<Cfg>(a, split_v, split_n, s);
        if (st != IREE_AMD_UK_STATUS_NOT_FOUND) return st;
      }
    }
  }
  // A last round that fills only part of the device costs a whole round. When
  // the large tile leaves such a round, the longer outer dimension is split:
  // whole rounds of 256x256 tiles first, the remaining rows or columns as a
  // second launch with whatever suits them (usually tiles of half the size, one
  // per compute unit). Taken when the model predicts at least 5 % (a launch costs a few
  // microseconds, so only for long K).
  const int64_t rows0 = ceil_div((int64_t)a.M, (int64_t)8);   // macro-tile rows of the large tile
  const int64_t cols0 = ceil_div((int64_t)a.N, (int64_t)8);
  const int64_t rounds0 = rows0 * cols0 / cus;
  if (rounds0 >= 1 && a.batch <= 1 && (int64_t)a.ksteps * Cfg::kMfmaK * Cfg::kElemBytes >= 2048) {
    // split the longer dimension: `across` macro tiles lie across it
    const bool by_cols = cols0 >= rows0;
    const int64_t across = by_cols ? rows0 : cols0;
    const int64_t along_first = rounds0 * cus / across;          // macro tiles along it in whole rounds
    const int64_t t_first = along_first * 8;                      // outer tiles
    const int64_t t_all = by_cols ? a.N : a.M;
    if (along_first >= 1 && t_first < t_all) {
      double rest_cost = 0;
      const int rest_v = by_cols ? pick(a.M, a.N - t_first, &rest_cost) : pick(a.M - t_first, a.N, &rest_cost);
      const double split_cost = (by_cols ? cost_of(0, a.M, t_first) : cost_of(0, t_first, a.N)) + rest_cost;
      if (split_cost < best_cost * 0.95) {
        MfmaArgs first = a, rest = a;
        const int64_t out_elem = kSiluMul ? 1 : (int64_t)sizeof(typename Cfg::out_t);
        if (by_cols) {
          first.N = (int)t_first;
          rest.N = a.N - (int)t_first;
          rest.rhs = a.rhs + t_first * a.rhs_stride_bytes;
          if (kSiluMul) {
            rest.out = a.out + (t_first / 2) * 1024;             // one e4m3 tile pair per two columns
          } else if (a.row_major_out) {
            rest.out = a.out + t_first * 32 * out_elem;
            first.out_cols = (int)(t_first * 32);                 // (out_cols > 32 (N - 1) >= 32 t_first)
            rest.out_cols = a.out_cols - (int)(t_first * 32);
          } else {
            rest.out = a.out + t_first * 1024 * out_elem;
          }
        } else {
          first.M = (int)t_first;
          rest.M = a.M - (int)t_first;
          // (tiled results and the SiLU form: out_stride_bytes is the pitch of an
          // outer row; row-major ones: of a matrix row)
          rest.out = a.out + t_first * (a.row_major_out ? 32 : 1) * a.out_stride_bytes;
          rest.lhs = a.lhs + t_first * (a.lhs_row_major ? 32 : 1) * a.lhs_stride_bytes;
          if (a.row_major_out) {
            first.out_rows = (int)(t_first * 32);
            rest.out_rows = a.out_rows - (int)(t_first * 32);
          }
        }
        const int st = launch(0, first);
        if (st) return st;
        return launch(rest_v, rest);
      }
    }
  }
  return launch(best, a);
}

}  // namespace
}  // namespace uk

#endif  // IREE_AMD_UK_MMT4D_MFMA_LAUNCH_H_
