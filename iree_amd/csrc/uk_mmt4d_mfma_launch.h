// Launch side of the matrix-core mmt4d kernels: the __global__ wrapper, the
// choice of the macro tile for a problem and the split of a partial last round.
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
  mmt4d_mfma_body<Cfg, WM, WN, kRing, kSync, kSiluMul, kWavesN, kForm>(a);
}

template <typename Cfg, int WM, int WN, int kRing, int kSync, int kOcc, bool kSiluMul, int kWavesN,
          int kForm>
int launch_form(const MfmaArgs& a, unsigned blocks, hipStream_t s) {
  constexpr int lds_bytes = mmt4d_mfma_lds_bytes<Cfg, WM, WN, kRing, kWavesN>();
  static_assert(lds_bytes <= 160 * 1024, "LDS ring exceeds 160 KiB");
  auto kernel = mmt4d_mfma_kernel<Cfg, WM, WN, kRing, kSync, kOcc, kSiluMul, kWavesN, kForm>;
  // The attribute belongs to the kernel on ONE device: set it once per device
  // ordinal (a benign race: the call is idempotent).
  static unsigned long long attr_set_on = 0;
  int dev = 0;
  UK_RETURN_IF_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64 || !((attr_set_on >> dev) & 1)) {
    UK_RETURN_IF_HIP(hipFuncSetAttribute((const void*)kernel,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes));
    if (dev >= 0 && dev < 64) attr_set_on |= 1ull << dev;
  }
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(128 * kWavesN), lds_bytes, s, a);
  return check_hip(hipGetLastError(), "mmt4d_mfma launch");
}

template <typename Cfg, int WM, int WN, int kRing, int kSync, int kOcc = 1, bool kSiluMul = false,
          int kWavesN = 2>
int launch_variant(const MfmaArgs& a0, hipStream_t s) {
  MfmaArgs a = a0;
  constexpr int kPerTile = 32 / Cfg::kRows;
  constexpr int TM = 2 * WM, TN = kWavesN * WN;   // blocks of Cfg::kRows rows
  static_assert(TM % kPerTile == 0 && TN % kPerTile == 0, "a workgroup covers whole outer tiles");
  a.tiles_m = (a.M * kPerTile + TM - 1) / TM;
  a.tiles_n = (a.N * kPerTile + TN - 1) / TN;
  const int64_t blocks = (int64_t)a.tiles_m * a.tiles_n;
  if (blocks > 0x7FFFFFFF) return IREE_AMD_UK_STATUS_NOT_FOUND;
  // one kernel instance per operand form (the forms the entry points produce)
  if constexpr (!kSiluMul) {
    if (a.lhs_row_major && a.row_major_out)
      return launch_form<Cfg, WM, WN, kRing, kSync, kOcc, kSiluMul, kWavesN, 2>(a, (unsigned)blocks, s);
    if (a.row_major_out)
      return launch_form<Cfg, WM, WN, kRing, kSync, kOcc, kSiluMul, kWavesN, 1>(a, (unsigned)blocks, s);
  }
  if (a.lhs_row_major || a.row_major_out) return IREE_AMD_UK_STATUS_NOT_FOUND;
  return launch_form<Cfg, WM, WN, kRing, kSync, kOcc, kSiluMul, kWavesN, 0>(a, (unsigned)blocks, s);
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
  auto cost_of = [&](int v, int64_t M, int64_t N) -> double {
    const Variant& t = variants[v];
    const int64_t tiles = ceil_div(M, (int64_t)2 * t.wm) * ceil_div(N, (int64_t)2 * t.wn);
    const int64_t slots = (int64_t)t.occ * cus;
    const double work = t.wm * t.wn;
    double cost = (double)(tiles / slots) * t.occ * work / t.eff_full;
    const int64_t rest = tiles % slots;
    if (rest > 0) {
      const int resident = (int)ceil_div(rest, (int64_t)cus);   // workgroups sharing a compute unit
      cost += resident * work / (resident == t.occ ? t.eff_full : t.eff_alone);
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
  auto launch = [&](int v, const MfmaArgs& b) -> int {
    switch (v) {
      case 0: return launch_variant<Cfg, 4 * S, 4 * S, kWide ? 5 : 8, kWide ? 1 : 2, 1, kSiluMul>(b, s);
      case 1: return launch_variant<Cfg, 4 * S, 2 * S, kWide ? 3 : 6, kWide ? 1 : 2, 2, kSiluMul>(b, s);
      case 2: return launch_variant<Cfg, 2 * S, 4 * S, kWide ? 3 : 6, kWide ? 1 : 2, 2, kSiluMul>(b, s);
      default: return launch_variant<Cfg, 2 * S, 2 * S, S == 2 ? 4 : 8, S == 2 ? 1 : 2, 1, kSiluMul>(b, s);
    }
  };
  double best_cost = 0;
  const int best = pick(a.M, a.N, &best_cost);
  // A last round that fills only part of the device costs a whole round. When
  // the large tile leaves such a round, the longer outer dimension is split:
  // whole rounds of 256x256 tiles first, the remaining rows or columns as a
  // second launch with whatever suits them (usually tiles of half the size, one
  // per compute unit). Taken when the model predicts at least 5 % (a launch costs a few
  // microseconds, so only for long K).
  const int64_t rows0 = ceil_div((int64_t)a.M, (int64_t)8);   // macro-tile rows of the large tile
  const int64_t cols0 = ceil_div((int64_t)a.N, (int64_t)8);
  const int64_t rounds0 = rows0 * cols0 / cus;
  if (rounds0 >= 1 && (int64_t)a.ksteps * Cfg::kMfmaK * Cfg::kElemBytes >= 2048) {
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
