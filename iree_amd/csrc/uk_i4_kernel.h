// The grouped int4-weight dequantising matmul kernel for workgroup slices of
// K = 512 KB (2048 or 4096; a last slice may be shorter), as a device function: wrapped in a __global__ by the library
// (uk_quant.hip, which describes the design) and by the code object built for a
// HAL executable.
#ifndef IREE_AMD_UK_I4_KERNEL_H_
#define IREE_AMD_UK_I4_KERNEL_H_

#include <type_traits>

#include "uk_i4.h"

namespace uk {
namespace i4 {
namespace {

// Work decomposition. A tile is 32 columns (n) of the output. Wave w of the
// workgroup owns k in [w*KB*64, (w+1)*KB*64), walked in KB/2 spans of 128: in
// one span lane (nl = l % 16, kc = l / 16) loads, for each half h of the
// tile's columns, 16 bytes of column h*16+nl, so that one wave load
// instruction moves a 16-column x 128-k slab (1 KiB, contiguous in the tiled
// layout). Its 4 dwords feed 4 MFMAs 16x16x32 (A = x rows m, B = weight
// columns n). Which k a dword holds depends on the layout: chunk (8 k) number
// q*4 + kc of the span in the tiled layout, kc*4 + q in the row-major one; the
// activation fragments are loaded to match (a.tiled), which in the tiled case
// makes each wave load of x cover 64 contiguous bytes of 16 rows.
//   MH       16-row halves of activations held (1: M <= 16, 2: M <= 32)
//   kZpU4    zero points are packed uint4 (else f16)
//   kLog2Gs  log2 of the group size, 5..8, or 9 for "at least the wave's K
//            slice" (one group per wave and tile). A group never straddles
//            MFMAs in the tiled layout (MFMA q covers k = q*32 .. +32 of the
//            span); in the row-major one that only holds for groups of 128
//            and more, so smaller groups are served from tiled weights only.
//   kStageX  (the 16-row form) the wave fetches its K slice of the activations
//            with one full-width direct-to-LDS load per row and takes its
//            operand fragments from there. Fetching them straight into the
//            operand layout costs 16 load instructions per wave whatever the
//            number of rows, and the kernel's start is bound by the rate at
//            which the compute unit takes load instructions (about 30 cycles
//            each, 8 waves): with one row the weights of the first tile are
//            requested 0.8 us earlier this way. Row r of a wave's staging
//            area is stored rotated by r chunks of 16 bytes (lane l fetches
//            chunk (l + r) mod row length), so that the 16 lanes that read one
//            chunk column of 16 rows hit 16 different bank groups without any
//            padding: 16 rows x 8 waves x 1 KiB are 128 KiB, which with the
//            32 KiB of partial sums is all the LDS there is. The area is sized
//            for 8 or for 16 rows (a.stage_rows). The 32-row form stages span
//            by span (128 k of all 32 rows at a time) through two buffers of
//            8 KiB per wave (the same 128 KiB, which its partial sums take
//            over afterwards), each span just ahead of the first tile's use
//            of it.
template <int N>
__device__ __forceinline__ void i4_wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

constexpr int kStageRowsMax = 16;
template <int KB>
constexpr int stage_row_bytes() { return KB * 128; }
constexpr int stage_rows_for(int rows) { return rows <= 8 ? 8 : 16; }

template <int KB, int MH, bool kZpU4, int kLog2Gs>
__device__ __forceinline__ void dequant_matmul_i4_body(const I4Args& a) {
  constexpr bool kStageX = MH == 1;
  constexpr int SP = KB / 2;                 // spans of 128 k per wave
  constexpr int L = kLog2Gs >= 9 ? 30 : kLog2Gs;
  constexpr int GW = ((KB * 64) >> L) > 0 ? ((KB * 64) >> L) : 1;   // groups per wave slice
  constexpr int SB = GW * 2;                 // bytes of scales per lane, tile and half
  constexpr int ZB = kZpU4 ? (GW >= 2 ? GW / 2 : 1) : GW * 2;
  constexpr int SW = (SB + 3) / 4, ZW = (ZB + 3) / 4;
  // Nibbles as f16 subnormals and the zero point applied through the group sums
  // of the activations (see nibbles_as_subnormals), where those sums fit the
  // register file: up to 8 accumulators of 4 registers, 16 in the 16-row form.
  constexpr bool kSubnormal = GW * MH <= 8 || (MH == 1 && GW <= 16);
  // Both forms stage the activations through dynamic LDS. The 16-row form keeps
  // the per-wave partial sums in static LDS next to it; in the 32-row form they
  // take over the staging area once the first tile has been multiplied.
  extern __shared__ __attribute__((aligned(16))) char stage_all[];
  typedef float Partial[kWaves][2 * MH * 4][64];
  Partial* partial;
  if constexpr (MH == 1) {
    __shared__ Partial partial_static[2];
    partial = partial_static;
  } else {
    partial = (Partial*)stage_all;
  }
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int nl = lane & 15, kc = lane >> 4;
  const int krow = blockIdx.y;               // K slice of this workgroup row (512 KB elements each)
  const int k_slice = (krow * kWaves + wave) * KB * 64;
  // A K that is not whole workgroup slices leaves the last waves of the last
  // workgroup row without any k (K is whole wave slices: the host checked).
  // Such a wave runs like the others on zeros: its loads of weights and
  // activations carry an offset past every buffer's end, which returns zeros
  // without touching memory, and its group parameters are those of the last
  // groups that exist (finite numbers, multiplied by sums that are zero).
  const bool wave_has_k = k_slice < a.K;
  const uint32_t past_end = wave_has_k ? 0u : 0x80000000u;
  int g_first = k_slice >> a.log2_gs;        // first group of this wave's slice
  {
    constexpr int kGroupsLoaded = ((KB * 64) >> (kLog2Gs >= 9 ? 30 : kLog2Gs)) > 0 ? ((KB * 64) >> (kLog2Gs >= 9 ? 30 : kLog2Gs)) : 1;
    if (!wave_has_k) g_first = a.G - kGroupsLoaded > 0 ? a.G - kGroupsLoaded : 0;
  }
  const uint32_t tile_bytes = (uint32_t)a.K * 16;
  const uint32_t voff = (nl * a.col_stride + kc * 16) | past_end;
  const uint32_t soff_wave = (krow * kWaves + wave) * SP * a.span_stride;
  const uint32_t half_stride = 16 * a.col_stride;

  // Raw group parameters of this lane's two columns for the wave's K slice
  // (zsh: position of a lone packed zero point inside its byte).
  struct Meta { uint32_t s[2][SW], z[2][ZW], zsh[2]; };
  // They are fetched with lane l % 32 taking column l % 32 of the tile, one
  // load instruction for the scales and one for the zero points of all 32
  // columns, and handed to the lanes that need them across the wave when the
  // tile begins (a compute unit takes a memory instruction only every 30 to 50
  // cycles whatever it moves: a load per column half, four per tile and wave
  // beside its eight of weights, was a third of the kernel's memory
  // instructions at one row).
  struct MetaRaw { uint32_t s[SW], z[ZW]; };
  auto load_meta = [&](int nt, MetaRaw& m) {
    int n = nt * 32 + (lane & 31);
    n = n < a.N ? n : a.N - 1;
    const size_t sg = (size_t)n * a.G + g_first;
    load_bits<SB>(a.scale + sg, m.s);
    if (kZpU4) load_bits<ZB>((const uint8_t*)a.zp + (sg >> 1), m.z);
    else load_bits<ZB>((const uint16_t*)a.zp + sg, m.z);
  };
  auto spread_meta = [&](const MetaRaw& raw, int nt) -> Meta {
    Meta m;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int from = (h * 16 + nl) * 4;       // (byte address of the source lane)
#pragma unroll
      for (int i = 0; i < SW; ++i) m.s[h][i] = (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)raw.s[i]);
#pragma unroll
      for (int i = 0; i < ZW; ++i) m.z[h][i] = (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)raw.z[i]);
      int n = nt * 32 + h * 16 + nl;
      n = n < a.N ? n : a.N - 1;
      const size_t sg = (size_t)n * a.G + g_first;
      m.zsh[h] = (kZpU4 && GW == 1) ? (uint32_t)(sg & 1) * 4 : 0;
    }
    return m;
  };
  // Weights of one tile: loads past the end of the buffer (a tile after the
  // last one, columns past N) return zeros without touching memory.
  auto tile_rsrc = [&](int nt) {
    const uint32_t off = (uint32_t)nt * tile_bytes;   // the host checked that this fits
    const uint32_t left = nt < a.n_tiles ? a.w_bytes - off : 0;   // (columns past N: the buffer ends)
    return __builtin_amdgcn_make_buffer_rsrc((void*)(a.w + off), 0, left, 0x00020000);
  };
  auto load_slab = [&](__amdgpu_buffer_rsrc_t rsrc, int sp, int h) -> u32x4 {
    // (non-temporal: the weights are read once; measured 9.2 -> 8.8 us at one row)
    return __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, soff_wave + sp * a.span_stride + h * half_stride, 2);
  };

  // ---- request the first tile's parameters, x and the first tile's weights --
  // Loads return in order, and a compute unit takes a load instruction only
  // every 30-50 cycles: with 8 waves each fetching 32 rows that is what bounds
  // the start of the kernel (every workgroup reads all of x, from L2: 256 KiB
  // at 32 rows). Both forms therefore fetch x with full-width direct-to-LDS
  // loads, one row of the wave's slice per instruction, request the first
  // tile's weights behind the first rows, and pick the rows out of LDS as MFMA
  // operand fragments. While the first tile multiplies, it requests slab by
  // slab the weights of the NEXT tile as it frees their registers.
  // activations: rows m_base + mh*16 + nl, this wave's K slice; rows past M
  // are zeros.
  int nt = blockIdx.x;
  MetaRaw meta_next;
  int meta_next_tile = nt < a.n_tiles ? nt : a.n_tiles - 1;
  load_meta(meta_next_tile, meta_next);
  u32x4 xraw[MH][SP][4];
  u32x4 wreg[SP][2];
  if constexpr (kStageX) {
    constexpr int kRowBytes = stage_row_bytes<KB>();
    constexpr int kLanesPerRow = KB * 8;                 // 16-byte chunks of a row's slice
    char* stage = stage_all + wave * a.stage_rows * kRowBytes;
    const int rows = a.M - a.m_base;                     // (at most 16: the host chose this form)
    const int cq = a.tiled ? 32 : 8, ckc = a.tiled ? 8 : 32;   // chunk strides in k
    const __amdgpu_buffer_rsrc_t rsrc = tile_rsrc(nt);
    // One direct-to-LDS load per row, as many as there are rows, nothing waited
    // for in between; then the first tile's weights; then the wait for the rows
    // only (loads return in order: all but the weight loads issued since).
    const __amdgpu_buffer_rsrc_t xsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(a.x + (size_t)a.m_base * a.K + (wave_has_k ? k_slice : 0)), 0, 0x7FFFFFFF, 0x00020000);
    if (lane < kLanesPerRow) {
#pragma unroll 1
      for (int r = 0; r < rows; ++r)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(xsrc, (__attribute__((address_space(3))) void*)(stage + r * kRowBytes), 16,
                                                 (((lane + r) & (kLanesPerRow - 1)) * 16) | past_end, r * a.K * 2, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int sp = 0; sp < SP; ++sp)
#pragma unroll
      for (int h = 0; h < 2; ++h) wreg[sp][h] = load_slab(rsrc, sp, h);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(SP * 2) : "memory");
    // (the wave reads only what it loaded itself: no barrier)
#pragma unroll
    for (int sp = 0; sp < SP; ++sp)
#pragma unroll
      for (int q = 0; q < 4; ++q) xraw[0][sp][q] = u32x4{0u, 0u, 0u, 0u};
    if (nl < rows) {
      const char* my_row = stage + nl * kRowBytes;
#pragma unroll
      for (int sp = 0; sp < SP; ++sp)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int chunk = (sp * 128 + q * cq + kc * ckc) >> 3;      // of 8 elements, within the slice
          xraw[0][sp][q] = *(const u32x4*)(my_row + ((chunk - nl) & (kLanesPerRow - 1)) * 16);
        }
    }
  }
  // 32 rows: SPAN by span (128 k of the wave's slice, 256 bytes of each of the
  // 32 rows = 8 KiB) through two buffers per wave, the same full-width loads
  // (4 rows per instruction) and rotated rows. The first tile walks its spans
  // in order, so span s of the activations is only needed when that tile gets
  // to span s: spans 0 and 1 and the first tile's weights are requested at
  // once, span s + 2 when span s has gone to registers, so that the first
  // tile multiplies span s while spans s + 1 and s + 2 arrive (staging all
  // rows up front, in four phases of 8 rows: 12.4 us at 32 rows, this way
  // 11.8). Timestamps inside the kernel show what bounds it: a compute unit's
  // 8 waves get a 1 KiB load accepted every 35 cycles or so (29 bytes per
  // clock), and the 256 KiB of activations plus 128 KiB of weights that each
  // compute unit pulls in are 5.6 us of that path. Rows past M lie past the
  // end of the buffer and read as zeros.
  constexpr int kSpanLoads = 8;                              // load instructions per span and wave
  constexpr int kSpanBytes = 32 * 256;
  char* const span_stage = stage_all + wave * 2 * kSpanBytes;
  const int span_cq = a.tiled ? 32 : 8, span_ckc = a.tiled ? 8 : 32;   // chunk strides in k
  const int x_rows = a.M - a.m_base < 32 ? a.M - a.m_base : 32;
  const __amdgpu_buffer_rsrc_t span_src = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(a.x + (size_t)a.m_base * a.K + (wave_has_k ? k_slice : 0)), 0,
      (uint32_t)(((int64_t)x_rows * a.K - (wave_has_k ? k_slice : 0)) * 2), 0x00020000);
  auto request_span = [&](int p) {
#pragma unroll
    for (int i = 0; i < kSpanLoads; ++i) {
      const int row = 4 * i + (lane >> 4);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          span_src, (__attribute__((address_space(3))) void*)(span_stage + (p & 1) * kSpanBytes + i * 1024), 16,
          (row * a.K * 2 + (((lane & 15) + row) & 15) * 16) | past_end, p * 256, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // Span p has landed when at most the loads issued behind it are outstanding
  // (loads return in order; a smaller count than the true one only waits longer).
  // The first tile's order of issue, SP = 4: spans 0, 1, the tile's 8 slabs;
  // [span 0 taken] span 2; [span 1 taken] span 3, then the next tile's slabs
  // as the tile consumes its own, those of span 0 first (held back until
  // span 3 has been requested: a span requested behind loads from memory
  // would only be seen to land after them). SP = 2: spans 0, 1, 4 slabs, then
  // the next tile's slabs as usual.
  auto wait_for_span = [&](int p) {
    constexpr int kW = SP * 2;
    static_assert(SP == 2 || SP == 4, "the counts below are those of two or four spans");
    if constexpr (SP == 4) {
      if (p == 0) i4_wait_vmcnt<kSpanLoads + kW>();          // span 1, the slabs
      else if (p == 1) i4_wait_vmcnt<kW + kSpanLoads>();     // the slabs, span 2
      else if (p == 2) i4_wait_vmcnt<kSpanLoads + 4>();      // span 3, next slabs of spans 0 and 1
      else i4_wait_vmcnt<6>();                               // next slabs of spans 0 to 2
    } else {
      if (p == 0) i4_wait_vmcnt<kSpanLoads + kW>();
      else i4_wait_vmcnt<kW + 2>();
    }
  };
  auto take_span = [&](int p, u32x4 (&raw)[MH][SP][4]) {
    const char* buf = span_stage + (p & 1) * kSpanBytes;
#pragma unroll
    for (int mh = 0; mh < MH; ++mh) {
      const int row = mh * 16 + nl;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int chunk = (q * span_cq + kc * span_ckc) >> 3;       // of 8 elements, within the span
        raw[mh][p][q] = *(const u32x4*)(buf + row * 256 + ((chunk - row) & 15) * 16);
      }
    }
    // the reads have left LDS before anything is loaded over them
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  };
  if constexpr (!kStageX) {
    static_assert(MH == 2, "the span-wise staging serves the 32-row form");
    const __amdgpu_buffer_rsrc_t rsrc = tile_rsrc(nt);
    request_span(0);
    if constexpr (SP > 1) request_span(1);
#pragma unroll
    for (int sp = 0; sp < SP; ++sp)
#pragma unroll
      for (int h = 0; h < 2; ++h) wreg[sp][h] = load_slab(rsrc, sp, h);
    __builtin_amdgcn_sched_barrier(0);
  }
  half8 xf[MH][SP][4];
  // (kSubnormal) the sum of the activations of row r (accumulator layout: every
  // column the same) over group g of this wave's K slice; complete when the
  // first tile reaches the end of the group, which is where it is used
  floatx4 xsum[kSubnormal ? MH : 1][kSubnormal ? GW : 1];
  if constexpr (kSubnormal) {
#pragma unroll
    for (int mh = 0; mh < MH; ++mh)
#pragma unroll
      for (int g = 0; g < GW; ++g) xsum[mh][g] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  int parity = 0;
  // One tile; `first`: the workgroup's first, which turns each span of x into
  // MFMA operands when it gets to it.
  auto tile = [&](auto first) {
    constexpr bool kFirst = decltype(first)::value;
    const int next = nt + gridDim.x;
    const Meta mt = spread_meta(meta_next, meta_next_tile);
    meta_next_tile = next < a.n_tiles ? next : a.n_tiles - 1;
    load_meta(meta_next_tile, meta_next);
    const __amdgpu_buffer_rsrc_t rsrc_next = tile_rsrc(next < a.n_tiles ? next : a.n_tiles);
    __builtin_amdgcn_sched_barrier(0);
    floatx4 acc[2][MH], part[2][MH];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int mh = 0; mh < MH; ++mh) acc[h][mh] = part[h][mh] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int sp = 0; sp < SP; ++sp) {
      if constexpr (kFirst && !kStageX) {
        __builtin_amdgcn_sched_barrier(0);
        wait_for_span(sp);
        take_span(sp, xraw);
        if (sp + 2 < SP) request_span(sp + 2);
        if (sp + 3 == SP) {
          // (the next tile's slabs of the spans before this one, held back so far)
#pragma unroll
          for (int e = 0; e < sp; ++e)
#pragma unroll
            for (int h = 0; h < 2; ++h) wreg[e][h] = load_slab(rsrc_next, e, h);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      if constexpr (kFirst) {
#pragma unroll
        for (int mh = 0; mh < MH; ++mh) {
          const uint32_t keep = kStageX || a.m_base + mh * 16 + nl < a.M ? 0xFFFFFFFFu : 0u;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            u32x4 v = xraw[mh][sp][q];
            if constexpr (!kStageX) { v.x &= keep; v.y &= keep; v.z &= keep; v.w &= keep; }
            if constexpr (kSubnormal) {
              xf[mh][sp][q] = permute_x_for_subnormals(v);
              const int g = (sp * 128 + q * 32) >> L;
              xsum[mh][g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[mh][sp][q], ones_for_subnormal_sums(),
                                                                  xsum[mh][g], 0, 0, 0);
            } else {
              xf[mh][sp][q] = permute_x(v);
            }
          }
        }
      }
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const u32x4 wv = wreg[sp][h];
        float sc = 0.f, zq = 0.f;
        union { uint32_t u; half2v h; } lo, hi, zf;
        lo.u = hi.u = zf.u = 0;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int k_lo = sp * 128 + q * 32;                 // within the wave's slice
          const int g = k_lo >> L;
          const bool group_start = kLog2Gs >= 9 ? k_lo == 0 : (k_lo & ((1 << L) - 1)) == 0;
          const bool group_end = kLog2Gs >= 9 ? k_lo + 32 == KB * 64 : ((k_lo + 32) & ((1 << L) - 1)) == 0;
          if (group_start || q == 0) {
            // decode the group's parameters
            const uint32_t sbits = (mt.s[h][g >> 1] >> ((g & 1) * 16)) & 0xFFFF;
            sc = __half2float(__ushort_as_half((uint16_t)sbits));
            if constexpr (kSubnormal) {
              // the products come in units of 2^-24; zq = -zp in those units
              sc *= kSubnormalRescale;
              if (kZpU4) {
                const uint32_t zb = (mt.z[h][g >> 3] >> ((g & 7) * 4 + mt.zsh[h])) & 0xF;
                zq = -(float)zb * kSubnormalUnit;
              } else {
                const uint32_t zb = (mt.z[h][g >> 1] >> ((g & 1) * 16)) & 0xFFFF;
                zq = -__half2float(__ushort_as_half((uint16_t)zb)) * kSubnormalUnit;
              }
            } else if (kZpU4) {
              // Packed uint4 zero points fold into the offsets (1024 + zp and
              // 64 + zp are exact). f16 zero points may carry a fraction, which
              // such a sum would round away: they are subtracted in a second step.
              const uint32_t zb = (mt.z[h][g >> 3] >> ((g & 7) * 4 + mt.zsh[h])) & 0xF;
              lo.u = offset_lo_bits(zb);
              hi.u = offset_hi_bits(zb);
            } else {
              const uint32_t zb = (mt.z[h][g >> 1] >> ((g & 1) * 16)) & 0xFFFF;
              lo.u = 0x64006400u;
              hi.h = half2v{(_Float16)64.0f, (_Float16)64.0f};
              zf.u = zb | (zb << 16);
            }
          }
          if (group_start) {
#pragma unroll
            for (int mh = 0; mh < MH; ++mh) part[h][mh] = floatx4{0.f, 0.f, 0.f, 0.f};
          }
          half8 wq;
          if constexpr (kSubnormal) {
            wq = nibbles_as_subnormals(wv[q]);
          } else {
            wq = dequant_dword(wv[q], lo.h, hi.h);
            if (!kZpU4) {
              const half8 zsub2 = {zf.h.x, zf.h.x, zf.h.x, zf.h.x, zf.h.x, zf.h.x, zf.h.x, zf.h.x};
              wq = wq - zsub2;
            }
          }
#pragma unroll
          for (int mh = 0; mh < MH; ++mh)
            part[h][mh] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[mh][sp][q], wq, part[h][mh], 0, 0, 0);
          if (group_end) {
#pragma unroll
            for (int mh = 0; mh < MH; ++mh)
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                float p = part[h][mh][r];
                if constexpr (kSubnormal) p = __builtin_fmaf(zq, xsum[mh][g][r], p);     // - zp * sum of x
                acc[h][mh][r] = __builtin_fmaf(p, sc, acc[h][mh][r]);
              }
          }
        }
        // The slab's registers are free: request the same slab of the next
        // tile. The fences keep the requests in slab order, which is what
        // makes every wait in the loop a wait for the OLDEST outstanding load.
        __builtin_amdgcn_sched_barrier(0);
        if (!(kFirst && !kStageX && sp + 3 < SP)) wreg[sp][h] = load_slab(rsrc_next, sp, h);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // ---- sum the 8 K-slices in wave order and store ----------------------
    float (*buf)[2 * MH * 4][64] = partial[parity];
    if constexpr (MH == 2 && kFirst) {
      // the partial sums overwrite the staging area: every wave has taken its
      // rows out of it by the time it gets here
      __builtin_amdgcn_s_barrier();
    }
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int mh = 0; mh < MH; ++mh)
#pragma unroll
        for (int r = 0; r < 4; ++r) buf[wave][(h * MH + mh) * 4 + r][lane] = acc[h][mh][r];
    __syncthreads();
#pragma unroll
    for (int rep = 0; rep < MH; ++rep) {
      const int flat = rep * kThreads + threadIdx.x;     // (h*MH + mh)*256 + r*64 + lane
      const int l = flat & 63, slot = flat >> 6;         // slot = (h*MH + mh)*4 + r
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) sum += buf[w][slot][l];
      const int r = slot & 3, hm = slot >> 2, h = hm / MH, mh = hm % MH;
      const int m = a.m_base + mh * 16 + 4 * (l >> 4) + r;
      const int n = nt * 32 + h * 16 + (l & 15);
      if (m < a.M && n < a.N) {
        if (a.partial) a.partial[((size_t)krow * a.M + m) * a.N + n] = sum;
        else a.out[(size_t)m * a.N + n] = __half_as_ushort(__float2half_rn(sum));
      }
    }
    // The other half of `partial` is used by the next tile; this half is
    // rewritten only two tiles later, after the next tile's barrier.
  };
  if (nt < a.n_tiles) {
    tile(std::true_type{});
    nt += gridDim.x;
    parity ^= 1;
  }
  for (; nt < a.n_tiles; nt += gridDim.x, parity ^= 1) tile(std::false_type{});
}

}  // namespace
}  // namespace i4
}  // namespace uk

#endif  // IREE_AMD_UK_I4_KERNEL_H_
