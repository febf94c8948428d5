// Grouped int4-weight dequantising matmul for up to 16 rows of activations and
// ANY K in whole 2048s (the kernel in uk_quant.hip keeps a slice of 2048 or
// 4096 of the activations in registers and takes a longer K as workgroup rows
// plus a second kernel that adds their sums; this one serves what that cannot
// take, and one row against few columns, where it measures faster). Same
// arithmetic, different decomposition:
//
//   * the activations (at most 16 rows) live in LDS, already in MFMA A-operand
//     order, shared by all waves of the workgroup;
//   * every WAVE owns whole output columns: a unit is 16 columns over all of K,
//     so there is no K split, no cross-wave reduction and no barrier after the
//     activations are staged;
//   * the weights of a unit are a stream of 1 KiB slabs (16 columns x 128 k)
//     through a rolling register buffer 16 slabs deep whose refills run ahead
//     across chunk and unit boundaries;
//   * K is walked in chunks of 2048 (16 slabs, fully unrolled, no predicates:
//     K is a whole number of chunks) with the group scales and zero points of
//     a chunk fetched one chunk ahead.
//
// When N is small (fewer units than waves on the device) the chunks of a unit
// are dealt to 2, 4 or 8 waves of the workgroup, which add their partial sums
// through LDS in a fixed order: a unit of K = 14336 then streams through 7
// waves at once instead of one.
//
// Measured against the K-split kernel where both apply (K = 4096, N = 14336,
// one row): 10.2 us against 10.1 us, and worse for small N, because one wave
// walks all of K for its columns alone (about 8 us of dependent latency and
// dequantisation); it is therefore used only for the K that kernel cannot take.
//
// The nibbles go to v_mfma_f32_16x16x32_f16 as f16 subnormals (one shift and
// four ANDs per 8 weights, every product exact in f32; uk_i4.h), the
// activations that meet the 16-fold pairs are divided by 16 when they are
// staged, the zero point multiplies the group's sum of activations, which a
// second MFMA against a constant operand takes alongside, and the per-group f32
// partial sums are scaled by the group's scale (the lane owns output column n,
// so scale and zero point are per-lane scalars).
#include "uk_common.h"
#include "uk_i4.h"

#include <memory>

namespace uk {
using namespace i4;
namespace {

constexpr int kChunkSpans = 16;   // 128-k spans per chunk (2048 k), unrolled
constexpr int kRingDepth = 16;    // slabs in flight per wave

struct GemvArgs {
  const uint16_t* x;      // [M][K] f16
  const uint8_t* w;
  const uint16_t* scale;  // [N][G]
  const uint8_t* zp;      // [N][G] f16 or packed u4
  uint16_t* out;          // [M][N] f16
  int M, N, K, G;
  int log2_gs;
  int tiled;
  int m_base, m_eff;      // rows of this pass: m_base .. m_base + m_eff (m_eff <= 16)
  int units;              // ceil(N / 16)
  int spans;              // K / 128
  int chunks;             // spans / 16
  int ksplit;             // waves that share one unit (1, 2, 4 or 8), each a range of chunks
  int chunks_per_part;    // chunks of one such wave (the last part may have fewer)
  int x_bytes;            // size of the staged activations in LDS (the partial sums follow)
  uint32_t w_bytes, scale_bytes, zp_bytes;
  // K split over workgroup rows (activations of all of K do not fit LDS):
  // row blockIdx.y owns chunks [y * row_chunks, ...) and writes f32 partial
  // sums [y][m][n] to partial_out; k_rows == 1: all chunks, f16 result
  int k_rows, row_chunks;
  float* partial_out;
};

// kLog2Gs: log2 of the group size for 6..8; 9 stands for "512 or more" (group
// boundaries are then tested at run time).
template <bool kZpU4, int kLog2Gs>
__global__ __launch_bounds__(kThreads) void dequant_gemv_i4_kernel(GemvArgs a) {
  constexpr bool kRuntimeGroups = kLog2Gs >= 9;
  constexpr int GC = kRuntimeGroups ? 0 : (2048 >> kLog2Gs);   // groups per chunk: 32, 16 or 8
  constexpr int SW = kRuntimeGroups ? 1 : GC / 8;              // u32x4 of scales per chunk
  constexpr int ZW = kRuntimeGroups ? 1 : (kZpU4 ? (GC >= 32 ? GC / 32 : 1) : GC / 8);
  extern __shared__ __attribute__((aligned(16))) char x_lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int nl = lane & 15, kc = lane >> 4;
  const int gs = 1 << a.log2_gs;

  // ---- flat sequence of (unit, chunk) pairs of this wave --------------------
  // Units go to workgroups first, then to waves, so that a small N still
  // spreads over all compute units.
  // With ksplit > 1, wave w is part w % ksplit of unit lane w / ksplit.
  const int kp = wave % a.ksplit, ulane = wave / a.ksplit;
  const int unit_lanes = kWaves / a.ksplit;
  const int unit0 = blockIdx.x + ulane * gridDim.x;
  const int unit_step = gridDim.x * unit_lanes;
  const int n_units = unit0 < a.units ? (a.units - unit0 + unit_step - 1) / unit_step : 0;
  // (chunk indices below are local to this workgroup row's K range)
  const int chunk_base = blockIdx.y * a.row_chunks;
  const int my_chunks = a.chunks - chunk_base < a.row_chunks ? a.chunks - chunk_base : a.row_chunks;
  int c0 = kp * a.chunks_per_part;
  c0 = c0 < my_chunks ? c0 : my_chunks;
  int c1 = c0 + a.chunks_per_part;
  c1 = c1 < my_chunks ? c1 : my_chunks;
  const int n_pairs = n_units * (c1 - c0);
  // parts that own chunks, and the unit rounds of the workgroup (unit lane 0
  // has the most): every wave meets that many barriers when ksplit > 1
  const int parts_used = (my_chunks + a.chunks_per_part - 1) / a.chunks_per_part;
  const int rounds = ((int)blockIdx.x < a.units) ? (a.units - (int)blockIdx.x + unit_step - 1) / unit_step : 0;

  const uint32_t span_stride = a.tiled ? 2048u : 64u;
  const uint32_t col_stride = a.tiled ? 64u : (uint32_t)(a.K >> 1);
  // Weights of a unit: a buffer whose end clips what lies beyond it to zeros
  // (columns past N of row-major weights, spans past K of tiled ones).
  auto unit_rsrc = [&](int unit) {
    uint32_t off, size;
    if (a.tiled) {
      off = (uint32_t)(unit >> 1) * ((uint32_t)a.K * 16) + (uint32_t)(unit & 1) * 1024u;
      size = (uint32_t)a.K * 16 - (uint32_t)(unit & 1) * 1024u;
    } else {
      off = (uint32_t)unit * 16u * col_stride;
      size = a.w_bytes - off;
    }
    if (unit >= a.units) size = 0;
    return __builtin_amdgcn_make_buffer_rsrc((void*)(a.w + off), 0, size, 0x00020000);
  };
  const uint32_t w_voff = nl * col_stride + kc * 16;
  // (the whole offset goes into the vector operand: that is the part the
  // hardware's range check is documented to cover)
  auto load_slab = [&](__amdgpu_buffer_rsrc_t rsrc, int span) -> u32x4 {
    return __builtin_amdgcn_raw_buffer_load_b128(rsrc, w_voff + (uint32_t)span * span_stride, 0, 2);   // (non-temporal: read once)
  };
  const __amdgpu_buffer_rsrc_t scale_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)a.scale, 0, a.scale_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t zp_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)a.zp, 0, a.zp_bytes, 0x00020000);
  // Group parameters of this lane's column for one chunk, as raw bits.
  struct Meta { u32x4 s[SW], z[ZW]; };
  auto load_meta = [&](int unit, int chunk, Meta& m) {
    if constexpr (!kRuntimeGroups) {
      int n = unit * 16 + nl;
      n = n < a.N ? n : a.N - 1;
      const uint32_t g0 = (uint32_t)n * a.G + (uint32_t)(chunk_base + chunk) * GC;     // first group of the chunk
#pragma unroll
      for (int i = 0; i < SW; ++i)
        m.s[i] = __builtin_amdgcn_raw_buffer_load_b128(scale_rsrc, g0 * 2 + i * 16, 0, 0);
      if constexpr (kZpU4) {
        if constexpr (GC >= 32) {
#pragma unroll
          for (int i = 0; i < ZW; ++i)
            m.z[i] = __builtin_amdgcn_raw_buffer_load_b128(zp_rsrc, g0 / 2 + i * 16, 0, 0);
        } else {   // 16 groups: 8 bytes, 8 groups: 4 bytes
          m.z[0].x = __builtin_amdgcn_raw_buffer_load_b32(zp_rsrc, g0 / 2, 0, 0);
          if constexpr (GC == 16) m.z[0].y = __builtin_amdgcn_raw_buffer_load_b32(zp_rsrc, g0 / 2 + 4, 0, 0);
        }
      } else {
#pragma unroll
        for (int i = 0; i < ZW; ++i)
          m.z[i] = __builtin_amdgcn_raw_buffer_load_b128(zp_rsrc, g0 * 2 + i * 16, 0, 0);
      }
    }
  };
  auto word_of = [](const u32x4* v, int i) -> uint32_t { return v[i >> 2][i & 3]; };

  // ---- stage x, then request the first slabs and parameters ----------------
  // x -> LDS in MFMA A-operand order: the 16 bytes that lane (row m, kc) feeds
  // MFMA number `step` (= span * 4 + q) lie at ((step * 4 + kc) * m_eff + m) * 16,
  // permuted to the k order of the weight dwords. Which 8 k those are depends
  // on the weight layout (see the other kernel): chunk q*4+kc of the span for
  // tiled weights, kc*4+q for row-major ones.
  // The activations go first, four loads in flight per thread: loads return in
  // order, so behind the 16 slabs of weights (which come from HBM) every round
  // of this loop would wait for all of them, and the loop is what the barrier
  // below waits for. (Measured inside the kernel at one row, K = 14336: staged
  // at 5.4 us with the weights requested first.)
  {
    const int chunks_per_row = my_chunks * 256;        // 8-element pieces of this row's K range
    const int total = a.m_eff * chunks_per_row;
    constexpr int kBatch = 4;
    for (int c0x = threadIdx.x; c0x < total; c0x += kThreads * kBatch) {
      u32x4 v[kBatch];
#pragma unroll
      for (int b = 0; b < kBatch; ++b) {
        const int c = c0x + b * kThreads;
        v[b] = u32x4{0u, 0u, 0u, 0u};
        if (c < total) {
          const int m = c / chunks_per_row, kchunk = c - m * chunks_per_row;
          v[b] = *(const u32x4*)(a.x + (size_t)(a.m_base + m) * a.K + (size_t)chunk_base * 2048 + kchunk * 8);
        }
      }
#pragma unroll
      for (int b = 0; b < kBatch; ++b) {
        const int c = c0x + b * kThreads;
        if (c < total) {
          const int m = c / chunks_per_row, kchunk = c - m * chunks_per_row;
          const int span = kchunk >> 4, r = kchunk & 15;
          const int q = a.tiled ? (r >> 2) : (r & 3), kcc = a.tiled ? (r & 3) : (r >> 2);
          union { half8 h; u32x4 u; } p;
          p.h = permute_x_for_subnormals(v[b]);
          *(u32x4*)(x_lds + (((span * 4 + q) * 4 + kcc) * a.m_eff + m) * 16) = p.u;
        }
      }
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  u32x4 ring[kRingDepth];
  Meta meta_next;
  {
    const __amdgpu_buffer_rsrc_t r0 = unit_rsrc(n_pairs > 0 ? unit0 : a.units);
    if (n_pairs > 0) load_meta(unit0, c0, meta_next);
#pragma unroll
    for (int d = 0; d < kRingDepth; ++d) ring[d] = load_slab(r0, (chunk_base + c0) * kChunkSpans + d);
  }
  __builtin_amdgcn_sched_barrier(0);
  __syncthreads();
  // Lanes of rows past m_eff read the last row: a row of A only reaches the
  // same row of the result, and those rows are never stored.
  const char* x_lane = x_lds + (kc * a.m_eff + (nl < a.m_eff ? nl : a.m_eff - 1)) * 16;
  const int x_step_bytes = 4 * a.m_eff * 16;

  // `part`: the products of the open group in units of 2^-24 (the nibbles are
  // f16 subnormals, see nibbles_as_subnormals); `xs`: the sum of the group's
  // activations, taken by a second MFMA against a constant operand (every
  // column the same), which is what the zero point multiplies.
  floatx4 acc = {0.f, 0.f, 0.f, 0.f}, part = {0.f, 0.f, 0.f, 0.f}, xs = {0.f, 0.f, 0.f, 0.f};
  float run_scale = 0.f, run_zq = 0.f;         // kRuntimeGroups: parameters of the open group
  const half8 ones = ones_for_subnormal_sums();
  floatx4* partial = (floatx4*)(x_lds + a.x_bytes);   // [2][kWaves][64], ksplit > 1 only
  int unit = unit0, chunk = c0, parity = 0;
  for (int pair = 0; pair < n_pairs; ++pair) {
    // the pair after this one (for the refills and the parameter prefetch)
    int next_unit = unit, next_chunk = chunk + 1;
    if (next_chunk == c1) { next_chunk = c0; next_unit = unit + unit_step; }
    const bool have_next = pair + 1 < n_pairs;
    const __amdgpu_buffer_rsrc_t rsrc_next = unit_rsrc(have_next ? next_unit : a.units);
    const Meta mt = meta_next;
    if (have_next) load_meta(next_unit, next_chunk, meta_next);
    __builtin_amdgcn_sched_barrier(0);
    const int span0 = chunk * kChunkSpans;
    int n = unit * 16 + nl;
    n = n < a.N ? n : a.N - 1;
    const char* x_chunk = x_lane + span0 * 4 * x_step_bytes;
#pragma unroll
    for (int s = 0; s < kChunkSpans; ++s) {
      const u32x4 wv = ring[s % kRingDepth];
      float sc = 0.f, zq = 0.f;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int k_in_chunk = s * 128 + q * 32;
        bool group_start, group_end;
        if constexpr (kRuntimeGroups) {
          const int k_abs = (chunk_base * kChunkSpans + span0) * 128 + k_in_chunk;
          group_start = (k_abs & (gs - 1)) == 0;
          group_end = ((k_abs + 32) & (gs - 1)) == 0;
          if (group_start) {
            const uint32_t sg = (uint32_t)n * a.G + (uint32_t)(k_abs >> a.log2_gs);
            const uint32_t sbits = __builtin_amdgcn_raw_buffer_load_b32(scale_rsrc, (sg * 2) & ~3u, 0, 0);
            run_scale = __half2float(__ushort_as_half((uint16_t)(sbits >> ((sg & 1) * 16)))) * kSubnormalRescale;
            if (kZpU4) {
              const uint32_t zw = __builtin_amdgcn_raw_buffer_load_b32(zp_rsrc, (sg >> 1) & ~3u, 0, 0);
              const uint32_t zb = (zw >> (((sg >> 1) & 3) * 8 + (sg & 1) * 4)) & 0xF;
              run_zq = -(float)zb * kSubnormalUnit;
            } else {
              const uint32_t zw = __builtin_amdgcn_raw_buffer_load_b32(zp_rsrc, (sg * 2) & ~3u, 0, 0);
              const uint32_t zb = (zw >> ((sg & 1) * 16)) & 0xFFFF;
              run_zq = -__half2float(__ushort_as_half((uint16_t)zb)) * kSubnormalUnit;
            }
          }
          sc = run_scale; zq = run_zq;
        } else {
          constexpr int L = kLog2Gs;
          const int g = k_in_chunk >> L;                 // group within the chunk
          group_start = (k_in_chunk & ((1 << L) - 1)) == 0;
          group_end = ((k_in_chunk + 32) & ((1 << L) - 1)) == 0;
          if (group_start || q == 0) {
            // the group's scale, times 2^24, and minus its zero point in units of 2^-24
            const uint32_t sbits = (word_of(mt.s, g >> 1) >> ((g & 1) * 16)) & 0xFFFF;
            sc = __half2float(__ushort_as_half((uint16_t)sbits)) * kSubnormalRescale;
            if (kZpU4) {
              const uint32_t zb = (word_of(mt.z, g >> 3) >> ((g & 7) * 4)) & 0xF;
              zq = -(float)zb * kSubnormalUnit;
            } else {
              const uint32_t zb = (word_of(mt.z, g >> 1) >> ((g & 1) * 16)) & 0xFFFF;
              zq = -__half2float(__ushort_as_half((uint16_t)zb)) * kSubnormalUnit;
            }
          }
        }
        if (group_start) {
          part = floatx4{0.f, 0.f, 0.f, 0.f};
          xs = floatx4{0.f, 0.f, 0.f, 0.f};
        }
        const half8 wq = nibbles_as_subnormals(wv[q]);
        union { half8 h; u32x4 u; } xa;
        xa.u = *(const u32x4*)(x_chunk + (s * 4 + q) * x_step_bytes);
        part = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa.h, wq, part, 0, 0, 0);
        xs = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa.h, ones, xs, 0, 0, 0);
        if (group_end) {
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[r] = __builtin_fmaf(__builtin_fmaf(zq, xs[r], part[r]), sc, acc[r]);
        }
      }
      // The slab's registers are free: request the slab kRingDepth further on,
      // in this chunk, the next one, or the next unit's first. The fences keep
      // the requests in stream order, so that every wait in the loop is a wait
      // for the oldest outstanding load.
      __builtin_amdgcn_sched_barrier(0);
      static_assert(kRingDepth == kChunkSpans, "a refill always lands in the next chunk");
      ring[s % kRingDepth] = load_slab(rsrc_next, (chunk_base + next_chunk) * kChunkSpans + s);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (chunk + 1 == c1) {
      // this wave's part of the unit is complete
      if (a.ksplit > 1) {
        // Sum the parts in part order (deterministic) in the wave of part 0.
        // The buffer alternates between units: a wave can only be one barrier
        // ahead of the reader of the previous unit's half.
        floatx4* buf = partial + parity * (kWaves * 64);
        buf[wave * 64 + lane] = acc;
        __syncthreads();
        if (kp == 0) {
          acc = buf[wave * 64 + lane];
          for (int p = 1; p < parts_used; ++p) {
            const floatx4 v = buf[(wave + p) * 64 + lane];
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[r] += v[r];
          }
        }
        parity ^= 1;
      }
      if (kp == 0) {
        // rows 4*kc + r of column n
        const int ncol = unit * 16 + nl;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int m = 4 * kc + r;
          if (m < a.m_eff && ncol < a.N) {
            if (a.k_rows > 1)
              a.partial_out[((size_t)blockIdx.y * a.m_eff + m) * a.N + ncol] = acc[r];
            else
              a.out[(size_t)(a.m_base + m) * a.N + ncol] = __half_as_ushort(__float2half_rn(acc[r]));
          }
        }
      }
      acc = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    unit = next_unit;
    chunk = next_chunk;
  }
  if (a.ksplit > 1) {
    // waves with fewer units than unit lane 0 (or without chunks) still meet
    // the barriers of the remaining rounds
    const int met = c1 > c0 ? n_units : 0;
    for (int r = met; r < rounds; ++r) __syncthreads();
  }
}

template <bool kZpU4>
int launch_zp(const GemvArgs& a, int blocks, size_t lds, hipStream_t s) {
  const dim3 g(blocks, a.k_rows), b(kThreads);
  // (once per kernel would do; the call is cheap and idempotent)
  auto set_lds = [&](const void* fn) {
    return hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
  };
  switch (a.log2_gs) {
    case 6: {
      auto k = dequant_gemv_i4_kernel<kZpU4, 6>;
      UK_RETURN_IF_HIP(set_lds((const void*)k));
      hipLaunchKernelGGL(k, g, b, lds, s, a);
      break;
    }
    case 7: {
      auto k = dequant_gemv_i4_kernel<kZpU4, 7>;
      UK_RETURN_IF_HIP(set_lds((const void*)k));
      hipLaunchKernelGGL(k, g, b, lds, s, a);
      break;
    }
    case 8: {
      auto k = dequant_gemv_i4_kernel<kZpU4, 8>;
      UK_RETURN_IF_HIP(set_lds((const void*)k));
      hipLaunchKernelGGL(k, g, b, lds, s, a);
      break;
    }
    default:
      return IREE_AMD_UK_STATUS_NOT_FOUND;
  }
  return check_hip(hipGetLastError(), "dequant_gemv_i4 launch");
}

}  // namespace

// Serves rows [m_base, m_base + m_eff) of the matmul, m_eff <= 16. Returns
// NOT_FOUND for shapes this kernel does not take (the caller then falls back).
int launch_dequant_gemv_i4(const I4Args& p, int m_base, int m_eff, hipStream_t s) {
  const int64_t K = p.K, N = p.N;
  const int64_t gs = 1ll << p.log2_gs;
  // K in whole chunks of 2048 (which also keeps every parameter vector of a
  // chunk 4-byte aligned), power-of-two groups of 64 and more (below 128 only
  // from tiled weights, where a group never straddles an MFMA), activations
  // that fit LDS.
  if (K % 2048 || m_eff < 1 || m_eff > 16) return IREE_AMD_UK_STATUS_NOT_FOUND;
  if (gs < (p.tiled ? 64 : 128) || gs > 256) return IREE_AMD_UK_STATUS_NOT_FOUND;
  const int64_t g_total = N * p.G;
  if (N * K / 2 + K * 16 >= (1ll << 32) || g_total * 2 >= (1ll << 32)) return IREE_AMD_UK_STATUS_NOT_FOUND;
  GemvArgs a;
  a.x = p.x; a.w = p.w; a.scale = p.scale; a.zp = (const uint8_t*)p.zp; a.out = p.out;
  a.M = p.M; a.N = p.N; a.K = p.K; a.G = p.G;
  a.log2_gs = p.log2_gs; a.tiled = p.tiled;
  a.m_base = m_base; a.m_eff = m_eff;
  a.units = (int)ceil_div(N, (int64_t)16);
  a.spans = (int)(K / 128);
  a.chunks = a.spans / kChunkSpans;
  a.w_bytes = (uint32_t)(N * K / 2);
  a.scale_bytes = (uint32_t)(g_total * 2);
  a.zp_bytes = (uint32_t)(p.zp_u4 ? (g_total + 1) / 2 : g_total * 2);
  // The activations of a workgroup's K range live in LDS (144 KiB of it). When
  // those of all of K do not fit, K is split over workgroup rows: every row
  // writes f32 partial sums to the stream's scratch buffer and the K-split
  // reduction kernel adds them in row order and rounds to f16 once.
  const int64_t chunk_x_bytes = (int64_t)m_eff * 2048 * 2;
  a.row_chunks = a.chunks;
  a.k_rows = 1;
  a.partial_out = nullptr;
  std::unique_ptr<ScratchLease> lease;   // held until the reduction has been queued
  if (a.chunks * chunk_x_bytes > 144 * 1024) {
    a.row_chunks = (int)((144 * 1024) / chunk_x_bytes);
    if (a.row_chunks < 1 || N % 4) return IREE_AMD_UK_STATUS_NOT_FOUND;
    a.k_rows = (a.chunks + a.row_chunks - 1) / a.row_chunks;
    a.row_chunks = (a.chunks + a.k_rows - 1) / a.k_rows;      // equal rows
    a.k_rows = (a.chunks + a.row_chunks - 1) / a.row_chunks;
    lease.reset(new ScratchLease(s, (size_t)a.k_rows * m_eff * N * 4));
    a.partial_out = (float*)lease->ptr();
    if (!a.partial_out) return IREE_AMD_UK_STATUS_NOT_FOUND;
  }
  size_t lds = (size_t)(a.row_chunks * chunk_x_bytes);
  // Few units (small N): deal the chunks of a unit to several waves, as many
  // as still leave every wave of the device at most one part of one unit.
  const int cus = device_cu_count();
  a.ksplit = 1;
  while (a.ksplit < kWaves && (int64_t)a.units * a.k_rows * a.ksplit * 2 <= (int64_t)cus * kWaves &&
         a.ksplit < a.row_chunks)
    a.ksplit *= 2;
  a.chunks_per_part = (a.row_chunks + a.ksplit - 1) / a.ksplit;
  a.x_bytes = (int)lds;
  if (a.ksplit > 1) lds += 2 * kWaves * 64 * sizeof(floatx4);   // 16 KiB of partial sums
  // (units go to workgroups first, then to the unit lanes of a workgroup; with
  // K rows, a row gets its share of the compute units)
  int blocks = cus / a.k_rows;
  if (blocks < 1) blocks = 1;
  if (blocks > a.units) blocks = a.units;
  int st = p.zp_u4 ? launch_zp<true>(a, blocks, lds, s) : launch_zp<false>(a, blocks, lds, s);
  if (st || a.k_rows == 1) return st;
  KSplitReduceArgs r;
  r.partials = a.partial_out;
  r.slices = a.k_rows;
  r.M = 1; r.N = 1;
  r.flat_elems = (int64_t)m_eff * N;
  r.out = p.out + (size_t)m_base * N;
  r.out_stride_bytes = 0;
  r.accumulate = 0;
  r.row_major_out = 0; r.out_rows = r.out_cols = 0;
  r.out_scale = 1.0f;
  r.acc_is_float = 1;
  r.out_kind = 1;   // f16
  return launch_ksplit_reduce(r, s);
}

}  // namespace uk
