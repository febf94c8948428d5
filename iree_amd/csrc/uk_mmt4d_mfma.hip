// mmt4d on the gfx950 matrix cores.
//
// Contract: include/iree_amd_uk.h (mirrors iree_uk_mmt4d,
// runtime/src/iree/builtins/ukernel/mmt4d.h:14-21 of the reference). This file
// serves the tile shapes the gfx950 tile-size query hands out: M0 = N0 = 32 and
// a K0 such that one lane's MFMA operand (16 bytes) is one contiguous piece of a
// tile row:
//
//   type            MFMA                         K per MFMA   K0 served
//   f16 x f16 -> f32  v_mfma_f32_32x32x16_f16        16         8, 16
//   bf16 x bf16 -> f32 v_mfma_f32_32x32x16_bf16      16         8, 16
//   s8 x s8 -> s32    v_mfma_i32_32x32x32_i8         32         16, 32
//
// With K0 = half the MFMA's K extent, two consecutive K tiles of one outer row
// ARE one MFMA operand in register order (lane l <-> bytes [16 l, 16 l + 16)),
// so a 64-lane 128-bit load moves a 1 KiB operand block with perfectly linear
// addressing. With K0 = the full extent the same 1 KiB holds one tile and the
// lane <-> address map is (l % 32) * 32 + (l / 32) * 16.
//
// Kernel shape: a workgroup of 4 waves owns a macro tile of (2*WM) x (2*WN)
// outer tiles; each wave accumulates WM x WN blocks of 32x32 in registers. The K
// loop moves operand blocks global -> LDS with direct-to-LDS 128-bit loads
// (no register staging), double buffered: the loads of stage s+1 are in flight
// while the MFMAs of stage s issue. Workgroup ids are remapped so that the 8
// XCDs (which receive consecutive workgroup ids round-robin) each work on a
// compact block of macro tiles and reuse operand panels in their own L2.
#include "uk_common.h"

namespace uk {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef int int4v __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef int intx16 __attribute__((ext_vector_type(16)));

struct F16Cfg {
  typedef half8 frag_t;
  typedef floatx16 acc_t;
  typedef float out_t;
  static constexpr int kElemBytes = 2;
  static constexpr int kMfmaK = 16;
  __device__ static acc_t mfma(frag_t a, frag_t b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};
struct BF16Cfg {
  typedef bf16x8 frag_t;
  typedef floatx16 acc_t;
  typedef float out_t;
  static constexpr int kElemBytes = 2;
  static constexpr int kMfmaK = 16;
  __device__ static acc_t mfma(frag_t a, frag_t b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
struct S8Cfg {
  typedef int4v frag_t;
  typedef intx16 acc_t;
  typedef int32_t out_t;
  static constexpr int kElemBytes = 1;
  static constexpr int kMfmaK = 32;
  __device__ static acc_t mfma(frag_t a, frag_t b, acc_t c) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
  }
};

constexpr int kThreads = 256;
constexpr int kSteps = 4;           // MFMA K-steps per LDS stage
constexpr int kBlockBytes = 1024;   // one 32-row operand block of one K-step

struct MfmaArgs {
  const char* lhs;  // offset applied
  const char* rhs;
  char* out;
  int64_t lhs_stride_bytes, rhs_stride_bytes, out_stride_bytes;
  int M, N;          // outer tile counts
  int ksteps;        // number of MFMA K-steps = K * K0 / kMfmaK
  int tiles_m, tiles_n;  // macro-tile grid
  int accumulate;
};

__device__ __forceinline__ void load_block_to_lds(const char* gptr, char* lds) {
  // 64 lanes x 16 bytes -> lds[0..1024) in lane order; gptr is per lane.
  __builtin_amdgcn_global_load_lds(
      (const __attribute__((address_space(1))) void*)gptr,
      (__attribute__((address_space(3))) void*)lds, 16, 0, 0);
}

// Maps the hardware workgroup id to a macro-tile coordinate. Workgroup ids go
// round-robin over the 8 XCDs; give XCD x the x-th contiguous slice of the
// logical tile sequence, and order that sequence in column-panels of `kGroup`
// macro-tile rows so that a slice is a compact 2-D block.
__device__ __forceinline__ void tile_coord(int bid, int tiles_m, int tiles_n,
                                           int* tm, int* tn) {
  constexpr int kXcds = 8, kGroup = 4;
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

template <typename Cfg, int WM, int WN, bool kHalfK0>
__global__ __launch_bounds__(kThreads) void mmt4d_mfma_kernel(MfmaArgs a) {
  typedef typename Cfg::frag_t frag_t;
  typedef typename Cfg::acc_t acc_t;
  typedef typename Cfg::out_t out_t;
  constexpr int TM = 2 * WM, TN = 2 * WN;      // outer tiles per workgroup
  constexpr int kRowBytes = kSteps * kBlockBytes;  // one outer row, one stage
  constexpr int kABytes = TM * kRowBytes, kBBytes = TN * kRowBytes;
  constexpr int kStageBytes = kABytes + kBBytes;
  extern __shared__ __attribute__((aligned(1024))) char lds[];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  int tm, tn;
  tile_coord(blockIdx.x, a.tiles_m, a.tiles_n, &tm, &tn);
  const int i_base = tm * TM, j_base = tn * TN;

  // Per-lane byte offset inside a 1 KiB operand block in global memory.
  const int lane_off = kHalfK0 ? lane * 16 : ((lane & 31) * 32 + (lane >> 5) * 16);

  // Rows this wave copies each stage: TM/4 rows of A and TN/4 rows of B.
  // Out-of-range rows are clamped to the last valid one (loaded, never stored).
  constexpr int kARowsPerWave = TM / 4, kBRowsPerWave = TN / 4;
  const char* a_src[kARowsPerWave];
  const char* b_src[kBRowsPerWave];
#pragma unroll
  for (int r = 0; r < kARowsPerWave; ++r) {
    int i = i_base + wave * kARowsPerWave + r;
    i = i < a.M ? i : a.M - 1;
    a_src[r] = a.lhs + (int64_t)i * a.lhs_stride_bytes + lane_off;
  }
#pragma unroll
  for (int r = 0; r < kBRowsPerWave; ++r) {
    int j = j_base + wave * kBRowsPerWave + r;
    j = j < a.N ? j : a.N - 1;
    b_src[r] = a.rhs + (int64_t)j * a.rhs_stride_bytes + lane_off;
  }

  acc_t acc[WM][WN];
  if (a.accumulate) {
#pragma unroll
    for (int x = 0; x < WM; ++x)
#pragma unroll
      for (int y = 0; y < WN; ++y) {
        int i = i_base + wm * WM + x, j = j_base + wn * WN + y;
        i = i < a.M ? i : a.M - 1;
        j = j < a.N ? j : a.N - 1;
        const out_t* t = (const out_t*)(a.out + (int64_t)i * a.out_stride_bytes) + (int64_t)j * 1024;
#pragma unroll
        for (int v = 0; v < 16; ++v)
          acc[x][y][v] = t[(8 * (v >> 2) + 4 * (lane >> 5) + (v & 3)) * 32 + (lane & 31)];
      }
  } else {
#pragma unroll
    for (int x = 0; x < WM; ++x)
#pragma unroll
      for (int y = 0; y < WN; ++y)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[x][y][v] = 0;
  }

  // Copies this wave's share of one stage: `nsteps` K-steps starting at
  // K-step `ks0` for kARowsPerWave rows of A and kBRowsPerWave rows of B.
  auto issue_rows = [&](char* stage_base, int ks0, int s) {
    char* sa = stage_base;
    char* sb = stage_base + kABytes;
#pragma unroll
    for (int r = 0; r < kARowsPerWave; ++r)
      load_block_to_lds(a_src[r] + (int64_t)(ks0 + s) * kBlockBytes,
                        sa + (wave * kARowsPerWave + r) * kRowBytes + s * kBlockBytes);
#pragma unroll
    for (int r = 0; r < kBRowsPerWave; ++r)
      load_block_to_lds(b_src[r] + (int64_t)(ks0 + s) * kBlockBytes,
                        sb + (wave * kBRowsPerWave + r) * kRowBytes + s * kBlockBytes);
  };
  auto issue_full = [&](int stage, int ks0) {
#pragma unroll
    for (int s = 0; s < kSteps; ++s) issue_rows(lds + stage * kStageBytes, ks0, s);
  };
  auto issue_tail = [&](int stage, int ks0, int nsteps) {
#pragma unroll 1
    for (int s = 0; s < nsteps; ++s) issue_rows(lds + stage * kStageBytes, ks0, s);
  };

  // One K-step of this wave's WM x WN blocks out of the given stage.
  auto compute_step = [&](const char* stage_base, int s) {
    const char* sa = stage_base + (wm * WM) * kRowBytes + lane * 16 + s * kBlockBytes;
    const char* sb = stage_base + kABytes + (wn * WN) * kRowBytes + lane * 16 + s * kBlockBytes;
    frag_t fa[WM], fb[WN];
#pragma unroll
    for (int x = 0; x < WM; ++x) fa[x] = *(const frag_t*)(sa + x * kRowBytes);
#pragma unroll
    for (int y = 0; y < WN; ++y) fb[y] = *(const frag_t*)(sb + y * kRowBytes);
#pragma unroll
    for (int x = 0; x < WM; ++x)
#pragma unroll
      for (int y = 0; y < WN; ++y) acc[x][y] = Cfg::mfma(fa[x], fb[y], acc[x][y]);
  };
  auto compute_full = [&](int stage) {
#pragma unroll
    for (int s = 0; s < kSteps; ++s) compute_step(lds + stage * kStageBytes, s);
  };
  auto compute_tail = [&](int stage, int nsteps) {
#pragma unroll 1
    for (int s = 0; s < nsteps; ++s) compute_step(lds + stage * kStageBytes, s);
  };
  // All of this wave's direct-to-LDS loads have landed, and (after the
  // barrier) so have everybody else's; every wave has also left the stage that
  // is about to be overwritten.
  auto stage_fence = [&]() {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  };

  const int nfull = a.ksteps / kSteps;
  const int tail = a.ksteps - nfull * kSteps;
  if (nfull > 0) {
    issue_full(0, 0);
    for (int st = 0; st + 1 < nfull; ++st) {
      stage_fence();
      issue_full((st + 1) & 1, (st + 1) * kSteps);
      compute_full(st & 1);
    }
    stage_fence();
    if (tail) issue_tail(nfull & 1, nfull * kSteps, tail);
    compute_full((nfull - 1) & 1);
    if (tail) {
      stage_fence();
      compute_tail(nfull & 1, tail);
    }
  } else {
    issue_tail(0, 0, tail);
    stage_fence();
    compute_tail(0, tail);
  }

  // Epilogue. MFMA 32x32 accumulator layout: register v of lane l holds
  // row 8*(v/4) + 4*(l/32) + v%4, column l%32 of the block; one store
  // instruction therefore writes two full 128-byte rows of the tile.
#pragma unroll
  for (int x = 0; x < WM; ++x)
#pragma unroll
    for (int y = 0; y < WN; ++y) {
      const int i = i_base + wm * WM + x, j = j_base + wn * WN + y;
      if (i < a.M && j < a.N) {
        out_t* t = (out_t*)(a.out + (int64_t)i * a.out_stride_bytes) + (int64_t)j * 1024;
#pragma unroll
        for (int v = 0; v < 16; ++v)
          t[(8 * (v >> 2) + 4 * (lane >> 5) + (v & 3)) * 32 + (lane & 31)] = acc[x][y][v];
      }
    }
}

template <typename Cfg, int WM, int WN, bool kHalfK0>
int launch_variant(const MfmaArgs& a0, hipStream_t s) {
  MfmaArgs a = a0;
  constexpr int TM = 2 * WM, TN = 2 * WN;
  a.tiles_m = (a.M + TM - 1) / TM;
  a.tiles_n = (a.N + TN - 1) / TN;
  const int64_t blocks = (int64_t)a.tiles_m * a.tiles_n;
  if (blocks > 0x7FFFFFFF) return IREE_AMD_UK_STATUS_NOT_FOUND;
  constexpr int lds_bytes = 2 * (TM + TN) * kSteps * kBlockBytes;
  auto kernel = mmt4d_mfma_kernel<Cfg, WM, WN, kHalfK0>;
  static bool attr_set = false;  // benign race: the call is idempotent
  if (!attr_set) {
    UK_RETURN_IF_HIP(hipFuncSetAttribute((const void*)kernel,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes));
    attr_set = true;
  }
  hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(kThreads), lds_bytes, s, a);
  return check_hip(hipGetLastError(), "mmt4d_mfma launch");
}

template <typename Cfg>
int launch_cfg(const MfmaArgs& a, bool half_k0, hipStream_t s) {
  // Pick the macro tile: the largest one (best operand reuse) when it still
  // yields at least one workgroup per compute unit, else the smaller one.
  const int cus = device_cu_count();
  const int64_t big = (int64_t)((a.M + 7) / 8) * ((a.N + 7) / 8);
  if (big >= cus) {
    return half_k0 ? launch_variant<Cfg, 4, 4, true>(a, s) : launch_variant<Cfg, 4, 4, false>(a, s);
  }
  return half_k0 ? launch_variant<Cfg, 2, 2, true>(a, s) : launch_variant<Cfg, 2, 2, false>(a, s);
}

struct Served { int mfma_k; };
bool served(uint32_t flags, int M0, int N0, int K0, Served* out) {
  int mfma_k = 0;
  switch (flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK) {
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F32:
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16F32: mfma_k = 16; break;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32: mfma_k = 32; break;
    default: return false;
  }
  if (M0 != 32 || N0 != 32) return false;
  if (K0 != mfma_k && K0 * 2 != mfma_k) return false;
  if (out) out->mfma_k = mfma_k;
  return true;
}

}  // namespace

bool mmt4d_mfma_supported(uint32_t flags, int M0, int N0, int K0) {
  return served(flags, M0, N0, K0, nullptr);
}

int launch_mmt4d_mfma(const iree_amd_uk_mmt4d_params_t& p, hipStream_t s) {
  Served sv;
  if (!served(p.flags, p.M0, p.N0, p.K0, &sv)) return IREE_AMD_UK_STATUS_NOT_FOUND;
  Mmt4dTypeInfo ti;
  mmt4d_type_info(p.flags, &ti);
  const int eb = ti.lhs_bits / 8;
  const int64_t k_elems = p.K * p.K0;
  // Whole MFMA K-steps only, and every operand block must be 16-byte aligned.
  if (p.K == 0 || k_elems % sv.mfma_k) return IREE_AMD_UK_STATUS_NOT_FOUND;
  const char* lhs = (const char*)p.lhs_buffer + p.lhs_offset * eb;
  const char* rhs = (const char*)p.rhs_buffer + p.rhs_offset * eb;
  if (((uintptr_t)lhs | (uintptr_t)rhs) % 16) return IREE_AMD_UK_STATUS_NOT_FOUND;
  if ((p.lhs_stride0 * eb) % 16 || (p.rhs_stride0 * eb) % 16) return IREE_AMD_UK_STATUS_NOT_FOUND;
  if (k_elems / sv.mfma_k > 0x7FFFFFFF) return IREE_AMD_UK_STATUS_NOT_FOUND;
  MfmaArgs a;
  a.lhs = lhs; a.rhs = rhs;
  a.out = (char*)p.out_buffer + p.out_offset * ti.out_bytes;
  a.lhs_stride_bytes = p.lhs_stride0 * eb;
  a.rhs_stride_bytes = p.rhs_stride0 * eb;
  a.out_stride_bytes = p.out_stride0 * ti.out_bytes;
  a.M = (int)p.M; a.N = (int)p.N;
  a.ksteps = (int)(k_elems / sv.mfma_k);
  a.tiles_m = a.tiles_n = 0;
  a.accumulate = (p.flags & IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE) != 0;
  const bool half_k0 = p.K0 * 2 == sv.mfma_k;
  switch (p.flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK) {
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F32: return launch_cfg<F16Cfg>(a, half_k0, s);
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16F32: return launch_cfg<BF16Cfg>(a, half_k0, s);
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32: return launch_cfg<S8Cfg>(a, half_k0, s);
    default: return IREE_AMD_UK_STATUS_NOT_FOUND;
  }
}

}  // namespace uk
