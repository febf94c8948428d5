// The reassociated form of the grouped int4 dequantising matmul: the opt-in
// rewrite of the reference's
// compiler/src/iree/compiler/GlobalOptimization/FuseDequantizationMatmul.cpp:398-645,749-767
// ("introduces precision loss ... opt-in only", :746-748), which is where its
// s16 x u4 -> s32 mmt4d ukernel comes from
// (runtime/src/iree/builtins/ukernel/arch/x86_64/mmt4d_x86_64_avx512_vnni.c:210-294):
//
//   scale_x[m][g] = max_k |x[m][g][k]| / 32767         group_sum[m][g] = sum_k x[m][g][k]
//   q[m][g][k]    = fptosi(x[m][g][k] / scale_x[m][g])                     (16 bits)
//   acc[m][n][g]  = sum_k q[m][g][k] * w[n][g][k]                          (exact, 32 bits)
//   out[m][n]     = sum_g float(acc) * scale_x * s[n][g] - (zp[n][g] * s[n][g]) * group_sum
//
// all float steps in f32. Two kernels: the quantisation of the activations (one
// wave per row and group; done once, every workgroup of the matmul needs all of
// it) and the matmul. On the matrix cores a 16-bit activation is two signed
// 8-bit digits, q = 256 hi + (lo - 128) + 128 with hi = q >> 8 and
// lo = q & 255, so that
//   sum q w = 256 sum hi w + sum (lo - 128) w + 128 sum w .
// One v_mfma_i32_32x32x32_i8 multiplies 16 rows of hi digits (operand rows
// 0..15) and the same 16 rows of lo digits (rows 16..31) with 32 columns of
// weights over 32 k; both sums of an (m, n) pair land in the same lane, 8
// registers apart. sum w comes from v_dot4 on the operand the lane has built
// anyway. The weights only have to be split into nibbles - three vector
// instructions per eight weights instead of the twelve of the f16
// dequantisation - which is what this form buys on a GPU.
#include "uk_common.h"
#include "uk_i4.h"

namespace uk {
using namespace i4;
namespace {

typedef int int4v __attribute__((ext_vector_type(4)));

struct ReassocArgs {
  // quantised activations of the rows [m_base, m_base + 16 * mh_count) for the
  // matmul kernel, in matrix-core operand order:
  //   planes[(((mh * spans + span) * 4 + q) * 64 + lane) * 16 + b]
  // span: 128 k; q: quarter of the span (one instruction's 32 k); lane =
  // kh * 32 + d * 16 + row % 16 with d: 0 = hi digit, 1 = lo - 128; byte b
  // <-> k = 128 span + 32 q + 16 kh + 8 (b / 8) + 2 (b % 4) + (b % 8) / 4 (the
  // order in which the nibbles of two weight dwords come out of the split).
  // scale_t / sum_t: [G][32] (row m - m_base).
  uint8_t* planes;
  float* scale_t;
  float* sum_t;
  // the same in plain layouts: q [M][K], scale_x / group_sum [M][G] (all rows)
  int16_t* q_plain;
  float* scale_plain;
  float* sum_plain;
  int mh_count, spans;
};

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) v = fmaxf(v, __shfl_xor(v, d, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) v = __fadd_rn(v, __shfl_xor(v, d, 64));
  return v;
}

// One wave per (row, group). rows: rows of x handled by this launch, from row0.
__global__ __launch_bounds__(256) void quantize_groups_i16_kernel(const uint16_t* x, int M, int K, int G,
                                                                 int gs, int row0, int rows, ReassocArgs r) {
  const int lane = threadIdx.x & 63;
  const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (unit >= (int64_t)rows * G) return;
  const int m = row0 + (int)(unit / G), g = (int)(unit % G);
  const uint16_t* xs = x + (size_t)m * K + (size_t)g * gs;
  float mx = 0.f, sum = 0.f;
  for (int e = lane; e < gs; e += 64) {
    const float v = __half2float(__ushort_as_half(xs[e]));
    mx = fmaxf(mx, fabsf(v));
    sum = __fadd_rn(sum, v);
  }
  mx = wave_max(mx);
  sum = wave_sum(sum);
  const float sc = __fdiv_rn(mx, 32767.0f);
  if (lane == 0) {
    if (r.scale_plain) { r.scale_plain[(size_t)m * G + g] = sc; r.sum_plain[(size_t)m * G + g] = sum; }
    if (r.scale_t) { r.scale_t[g * 32 + (m - row0)] = sc; r.sum_t[g * 32 + (m - row0)] = sum; }
  }
  for (int e = lane; e < gs; e += 64) {
    const float v = __half2float(__ushort_as_half(xs[e]));
    const int q = sc > 0.f ? (int)__fdiv_rn(v, sc) : 0;      // (float -> int conversion truncates)
    if (r.q_plain) r.q_plain[(size_t)m * K + (size_t)g * gs + e] = (int16_t)q;
    if (r.planes) {
      const int k = g * gs + e;
      const int span = k >> 7, rr = k & 127, qq = rr >> 5, kh = (rr >> 4) & 1, c8 = (rr >> 3) & 1, j = rr & 7;
      const int b = c8 * 8 + (j & 1) * 4 + (j >> 1);
      const int mr = m - row0, mh = mr >> 4;
      const size_t at = ((((size_t)mh * r.spans + span) * 4 + qq) * 64 + kh * 32 + (mr & 15)) * 16 + b;
      r.planes[at] = (uint8_t)(q >> 8);
      r.planes[at + 16 * 16] = (uint8_t)((q & 255) - 128);     // (lane + 16: the lo digit's operand row)
    }
  }
}

// Element-wise form for every shape the matrix-core kernel does not take: one
// thread per output element, the reference's order of operations.
__global__ __launch_bounds__(256) void dequant_matmul_i4_reassoc_generic_kernel(I4Args a, ReassocArgs r, int gs) {
  const int64_t total = (int64_t)a.M * a.N;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int m = (int)(idx / a.N), n = (int)(idx - (int64_t)m * a.N);
    float acc_out = 0.f;
    for (int g = 0; g < a.G; ++g) {
      const size_t sg = (size_t)n * a.G + g;
      float zpv;
      if (a.zp_u4) {
        const uint8_t byte = ((const uint8_t*)a.zp)[sg >> 1];
        zpv = (float)((sg & 1) ? (byte >> 4) : (byte & 0xF));
      } else {
        zpv = __half2float(__ushort_as_half(((const uint16_t*)a.zp)[sg]));
      }
      const float sc = __half2float(__ushort_as_half(a.scale[sg]));
      int acc = 0;
      for (int kk = 0; kk < gs; ++kk) {
        const int k = g * gs + kk;
        const uint8_t byte = a.w[a.tiled ? tiled_byte_index(n, k, a.K) : ((size_t)n * a.K + k) >> 1];
        const int wv = (k & 1) ? (byte >> 4) : (byte & 0xF);
        acc += (int)r.q_plain[(size_t)m * a.K + k] * wv;
      }
      const float r1 = __fmul_rn(__fmul_rn((float)acc, r.scale_plain[(size_t)m * a.G + g]), sc);
      const float z1 = __fmul_rn(__fmul_rn(zpv, sc), r.sum_plain[(size_t)m * a.G + g]);
      acc_out = __fadd_rn(__fsub_rn(r1, z1), acc_out);
    }
    a.out[idx] = __half_as_ushort(__float2half_rn(acc_out));
  }
}

// The matmul on the matrix cores. A tile is 32 output columns; wave w of the 8
// owns k in [w * KB * 64, (w + 1) * KB * 64), walked in spans of 128. Per span,
// lane (c, kh) loads the 32 bytes of column c that hold the 16-byte chunks
// 2 kh and 2 kh + 1 (tiled weights: dword q of chunk j is k = 32 q + 8 j .. + 8
// of the span). Dword q of both chunks, split into even and odd nibbles, is
// the lane's B operand of the span's q-th v_mfma_i32_32x32x32_i8; the
// activation digits were stored in that byte order.
//   MH       16-row halves of activations (1: M <= 16, 2: M <= 32)
//   kLog2Gs  log2 of the group size: 7, 8, or 9 = the wave's whole K slice
template <int KB, int MH, bool kZpU4, int kLog2Gs>
__global__ __launch_bounds__(kThreads) void dequant_matmul_i4_reassoc_kernel(I4Args a, ReassocArgs ro) {
  constexpr int SP = KB / 2;                 // spans of 128 k per wave
  constexpr int L = kLog2Gs;
  static_assert(L >= 7 && (128 << (L - 7)) <= KB * 64, "a group is whole spans of one wave");
  constexpr int GW = (KB * 64) >> L;         // groups per wave slice
  constexpr int SPG = SP / GW;               // spans per group
  typedef int intx16 __attribute__((ext_vector_type(16)));
  // [0]: the group tables of the rows (scale_x, group sums), then the partial
  // results of the K slices, double buffered over the tiles
  extern __shared__ __attribute__((aligned(16))) char lds_raw[];
  const int G = a.G;
  float* tab_scale = (float*)lds_raw;                    // [G][32]
  float* tab_sum = tab_scale + G * 32;                   // [G][32]
  float (*partial)[kWaves][8 * MH][64] = (float (*)[kWaves][8 * MH][64])(tab_sum + G * 32);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col = lane & 31, kh = lane >> 5;
  const int k_slice = wave * KB * 64;
  const int g_first = k_slice >> L;
  const uint32_t tile_bytes = (uint32_t)a.K * 16;
  const uint32_t voff = col * a.col_stride + kh * 32;
  const uint32_t soff_wave = wave * SP * a.span_stride;

  // Group parameters of this lane's column for the wave's K slice, as floats.
  struct Meta { float s[GW], z[GW]; };
  auto load_meta = [&](int nt, Meta& m) {
    int n = nt * 32 + col;
    n = n < a.N ? n : a.N - 1;
#pragma unroll
    for (int gw = 0; gw < GW; ++gw) {
      const size_t sg = (size_t)n * G + g_first + gw;
      m.s[gw] = __half2float(__ushort_as_half(a.scale[sg]));
      if (kZpU4) {
        const uint8_t byte = ((const uint8_t*)a.zp)[sg >> 1];
        m.z[gw] = (float)((sg & 1) ? (byte >> 4) : (byte & 0xF));
      } else {
        m.z[gw] = __half2float(__ushort_as_half(((const uint16_t*)a.zp)[sg]));
      }
    }
  };
  auto tile_rsrc = [&](int nt) {
    const uint32_t off = (uint32_t)nt * tile_bytes;
    const uint32_t left = nt < a.n_tiles ? a.w_bytes - off : 0;
    return __builtin_amdgcn_make_buffer_rsrc((void*)(a.w + off), 0, left, 0x00020000);
  };
  auto load_chunk = [&](__amdgpu_buffer_rsrc_t rsrc, int sp, int c8) -> u32x4 {
    // (ordinary loads: a lane's two chunks share their cache lines with its
    // neighbours' and the second request must still find them)
    return __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff + c8 * 16, soff_wave + sp * a.span_stride, 0);
  };

  const int rows = a.M - a.m_base;      // activation rows of this pass (at most 16 MH)
  int nt = blockIdx.x;
  Meta meta_next;
  load_meta(nt < a.n_tiles ? nt : a.n_tiles - 1, meta_next);
  u32x4 wreg[SP][2];
  {
    const __amdgpu_buffer_rsrc_t rsrc = tile_rsrc(nt);
#pragma unroll
    for (int sp = 0; sp < SP; ++sp)
#pragma unroll
      for (int c8 = 0; c8 < 2; ++c8) wreg[sp][c8] = load_chunk(rsrc, sp, c8);
  }
  // activation digits of this wave's K slice: operand rows 0..15 the hi digits
  // of rows 16 mh .. + 16, rows 16..31 their lo digits
  int4v xd[MH][SP][4];
#pragma unroll
  for (int mh = 0; mh < MH; ++mh)
#pragma unroll
    for (int sp = 0; sp < SP; ++sp)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        xd[mh][sp][q] = *(const int4v*)(ro.planes +
                                        ((((size_t)mh * ro.spans + wave * SP + sp) * 4 + q) * 64 + lane) * 16);
  // (requested last: everything above is already on its way when the first
  // wait for these values comes)
  for (int i = threadIdx.x; i < G * 32; i += kThreads) {
    tab_scale[i] = ro.scale_t[i];
    tab_sum[i] = ro.sum_t[i];
  }
  __syncthreads();      // the group tables are in LDS

  int parity = 0;
  for (; nt < a.n_tiles; nt += gridDim.x, parity ^= 1) {
    const int next = nt + gridDim.x;
    const Meta mt = meta_next;
    load_meta(next < a.n_tiles ? next : a.n_tiles - 1, meta_next);
    const __amdgpu_buffer_rsrc_t rsrc_next = tile_rsrc(next < a.n_tiles ? next : a.n_tiles);
    __builtin_amdgcn_sched_barrier(0);
    // out[m][n] of this lane: column `col`, rows 16 mh + 8 (v / 4) + 4 kh + v % 4, v < 8
    float acc[MH][8];
#pragma unroll
    for (int mh = 0; mh < MH; ++mh)
#pragma unroll
      for (int v = 0; v < 8; ++v) acc[mh][v] = 0.f;
    intx16 sums[MH];
    uint32_t wsum = 0;
#pragma unroll
    for (int sp = 0; sp < SP; ++sp) {
      const int gw = sp / SPG;
      if (sp % SPG == 0) {
        wsum = 0;
#pragma unroll
        for (int mh = 0; mh < MH; ++mh)
#pragma unroll
          for (int v = 0; v < 16; ++v) sums[mh][v] = 0;
      }
      const u32x4 w0 = wreg[sp][0], w1 = wreg[sp][1];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int4v b = {(int)(w0[q] & 0x0F0F0F0Fu), (int)((w0[q] >> 4) & 0x0F0F0F0Fu),
                         (int)(w1[q] & 0x0F0F0F0Fu), (int)((w1[q] >> 4) & 0x0F0F0F0Fu)};
#pragma unroll
        for (int e = 0; e < 4; ++e) wsum = __builtin_amdgcn_udot4((uint32_t)b[e], 0x01010101u, wsum, false);
#pragma unroll
        for (int mh = 0; mh < MH; ++mh)
          sums[mh] = __builtin_amdgcn_mfma_i32_32x32x32_i8(xd[mh][sp][q], b, sums[mh], 0, 0, 0);
      }
      // the span's registers are free: request the same span of the next tile
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int c8 = 0; c8 < 2; ++c8) wreg[sp][c8] = load_chunk(rsrc_next, sp, c8);
      __builtin_amdgcn_sched_barrier(0);
      if (sp % SPG == SPG - 1) {
        // End of a group: the float steps, in the reference's order. The sum
        // of the column's weights over the group: this lane's half of k plus
        // the other half's (lane ^ 32).
        const int wterm = (int)((wsum + (uint32_t)__shfl_xor((int)wsum, 32, 64)) << 7);
        const float sc = mt.s[gw], zs = __fmul_rn(mt.z[gw], mt.s[gw]);
        const int g = g_first + gw;
#pragma unroll
        for (int mh = 0; mh < MH; ++mh)
#pragma unroll
          for (int vh = 0; vh < 2; ++vh) {
            // rows 16 mh + 8 vh + 4 kh + r of this pass; only those below M are
            // worth the arithmetic (one of eight for a single row)
            const int live = rows - (mh * 16 + vh * 8);       // wave-uniform
            if (live <= 0) continue;
            const floatx4 sx = *(const floatx4*)(tab_scale + g * 32 + mh * 16 + vh * 8 + kh * 4);
            const floatx4 sm = *(const floatx4*)(tab_sum + g * 32 + mh * 16 + vh * 8 + kh * 4);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              if (r >= live) break;
              const int v = vh * 4 + r;
              const int total = (sums[mh][v] << 8) + sums[mh][v + 8] + wterm;
              const float r1 = __fmul_rn(__fmul_rn((float)total, sx[r]), sc);
              const float z1 = __fmul_rn(zs, sm[r]);
              acc[mh][v] = __fadd_rn(__fsub_rn(r1, z1), acc[mh][v]);
            }
          }
      }
    }
    // ---- sum the 8 K-slices in wave order and store ----------------------
    float (*buf)[8 * MH][64] = partial[parity];
#pragma unroll
    for (int mh = 0; mh < MH; ++mh)
#pragma unroll
      for (int v = 0; v < 8; ++v) buf[wave][mh * 8 + v][lane] = acc[mh][v];
    __syncthreads();
#pragma unroll
    for (int rep = 0; rep < MH; ++rep) {
      const int flat = rep * kThreads + threadIdx.x;     // (mh * 8 + v) * 64 + lane
      const int l = flat & 63, slot = flat >> 6;
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) sum = __fadd_rn(sum, buf[w][slot][l]);
      const int v = slot & 7, mh = slot >> 3;
      const int m = a.m_base + mh * 16 + 8 * (v >> 2) + 4 * (l >> 5) + (v & 3);
      const int n = nt * 32 + (l & 31);
      if (m < a.M && n < a.N) a.out[(size_t)m * a.N + n] = __half_as_ushort(__float2half_rn(sum));
    }
    // (the other half of `partial` serves the next tile; this half is rewritten
    // two tiles later, after the next tile's barrier)
  }
}

template <int KB, int MH, bool kZpU4, int kLog2Gs>
int launch_instance(const I4Args& a, const ReassocArgs& r, int blocks, hipStream_t s) {
  // group tables + the double-buffered partial results of the 8 K slices
  const size_t lds = (size_t)a.G * 32 * 2 * sizeof(float) + (size_t)2 * kWaves * 8 * MH * 64 * sizeof(float);
  void (*kernel)(I4Args, ReassocArgs) = dequant_matmul_i4_reassoc_kernel<KB, MH, kZpU4, kLog2Gs>;
  if (lds > 64 * 1024) {
    static PerDeviceOnce attr_set_on;
    int dev = 0;
    UK_RETURN_IF_HIP(hipGetDevice(&dev));
    if (!attr_set_on.done(dev)) {
      UK_RETURN_IF_HIP(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
      attr_set_on.mark(dev);
    }
  }
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(kThreads), lds, s, a, r);
  return check_hip(hipGetLastError(), "dequant_matmul_i4_reassoc launch");
}

template <int KB, int MH, bool kZpU4>
int launch_one(const I4Args& a, const ReassocArgs& r, int blocks, hipStream_t s) {
  const int log2_gs = a.log2_gs > 9 ? 9 : a.log2_gs;
  if (log2_gs == 7) return launch_instance<KB, MH, kZpU4, 7>(a, r, blocks, s);
  if (log2_gs == 8) return launch_instance<KB, MH, kZpU4, 8>(a, r, blocks, s);
  if constexpr (KB == 8) return launch_instance<KB, MH, kZpU4, 9>(a, r, blocks, s);
  return IREE_AMD_UK_STATUS_NOT_FOUND;
}

unsigned quantize_blocks(int64_t rows, int64_t G) { return (unsigned)ceil_div(rows * G, (int64_t)4); }

}  // namespace

int launch_quantize_groups_i16(const void* x, void* q, void* scale_x, void* group_sum, int64_t M,
                               int64_t K, int64_t gs, hipStream_t s) {
  if (M * (K / gs) > 0x7FFFFFFFll * 4 || K > 0x7FFFFFFF || M > 0x7FFFFFFF)
    return fail(IREE_AMD_UK_STATUS_OUT_OF_RANGE, "quantize_groups_i16: sizes beyond 2^31");
  ReassocArgs r = {};
  r.q_plain = (int16_t*)q;
  r.scale_plain = (float*)scale_x;
  r.sum_plain = (float*)group_sum;
  const int G = (int)(K / gs);
  hipLaunchKernelGGL(quantize_groups_i16_kernel, dim3(quantize_blocks(M, G)), dim3(256), 0, s,
                     (const uint16_t*)x, (int)M, (int)K, G, (int)gs, 0, (int)M, r);
  return check_hip(hipGetLastError(), "quantize_groups_i16 launch");
}

int launch_dequant_matmul_i4_reassoc(const void* x, const void* w, const void* scale, const void* zp,
                                     void* out, int64_t M, int64_t N, int64_t K, int64_t group_size,
                                     uint32_t flags, hipStream_t s) {
  if (M > 0x7FFFFFFF || N > 0x7FFFFFFF || K > 0x7FFFFFFF)
    return fail(IREE_AMD_UK_STATUS_OUT_OF_RANGE, "dequant_matmul_i4: sizes beyond 2^31");
  const bool tiled = (flags & IREE_AMD_UK_FLAG_DEQUANT_MATMUL_W_TILED) != 0;
  if (tiled && (N % 32 || K % 128))
    return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT,
                "dequant_matmul_i4: tiled weights need N %% 32 == 0 and K %% 128 == 0");
  I4Args a;
  a.x = (const uint16_t*)x; a.w = (const uint8_t*)w; a.scale = (const uint16_t*)scale;
  a.zp = zp; a.out = (uint16_t*)out;
  a.M = (int)M; a.N = (int)N; a.K = (int)K; a.G = (int)(K / group_size);
  a.zp_u4 = (flags & IREE_AMD_UK_FLAG_DEQUANT_MATMUL_ZP_U4) != 0;
  a.tiled = tiled;
  a.n_tiles = (int)ceil_div(N, 32);
  a.m_base = 0;
  a.stage_rows = 0;
  a.log2_gs = 0;
  while ((1ll << a.log2_gs) < group_size) ++a.log2_gs;
  const bool gs_pow2 = (1ll << a.log2_gs) == group_size;
  a.span_stride = 2048u;
  a.col_stride = 64u;
  const int64_t kb = K / 512;
  const int64_t w_bytes = N * K / 2;
  a.w_bytes = (uint32_t)w_bytes;
  const int cus = device_cu_count();
  // Matrix-core kernel: tiled weights, K = 2048 or 4096, power-of-two groups
  // of whole spans inside one wave's K slice, 16-byte aligned operands.
  const bool fast = tiled && K % 512 == 0 && (kb == 4 || kb == 8) && gs_pow2 && group_size >= 128 &&
                    group_size <= kb * 64 && w_bytes + K * 16 < (1ll << 32) &&
                    ((uintptr_t)w % 16) == 0 && ((uintptr_t)scale % 16) == 0 && ((uintptr_t)zp % 16) == 0;
  if (fast) {
    const int spans = (int)(K / 128);
    const size_t plane_bytes = (size_t)2 * spans * 4 * 64 * 16;          // 2 row halves, both digits
    const size_t table_bytes = (size_t)a.G * 32 * sizeof(float);
    // (held until the last kernel that reads it has been queued)
    CallScratch lease(s, plane_bytes + 2 * table_bytes);
    if (lease.overflowed()) return scratch_overflow_status("dequant_matmul_i4: the quantised activations", plane_bytes + 2 * table_bytes);
    if (!lease.ptr()) return fail(8 /* RESOURCE_EXHAUSTED */, "dequant_matmul_i4: no scratch memory for the quantised activations");
    note_kernel_path("dequant_i4:reassociated");
    for (int m_base = 0; m_base < a.M; m_base += 32) {
      const int rows = a.M - m_base < 32 ? a.M - m_base : 32;
      ReassocArgs r = {};
      r.mh_count = rows > 16 ? 2 : 1;
      r.spans = spans;
      r.planes = (uint8_t*)lease.ptr();
      r.scale_t = (float*)(r.planes + plane_bytes);
      r.sum_t = r.scale_t + (size_t)a.G * 32;
      hipLaunchKernelGGL(quantize_groups_i16_kernel, dim3(quantize_blocks(rows, a.G)), dim3(256), 0, s,
                         a.x, a.M, a.K, a.G, (int)group_size, m_base, rows, r);
      UK_RETURN_IF_HIP(hipGetLastError());
      a.m_base = m_base;
      const int blocks = a.n_tiles < cus ? a.n_tiles : cus;
      int st;
      if (kb == 4) {
        st = r.mh_count == 2 ? (a.zp_u4 ? launch_one<4, 2, true>(a, r, blocks, s) : launch_one<4, 2, false>(a, r, blocks, s))
                             : (a.zp_u4 ? launch_one<4, 1, true>(a, r, blocks, s) : launch_one<4, 1, false>(a, r, blocks, s));
      } else {
        st = r.mh_count == 2 ? (a.zp_u4 ? launch_one<8, 2, true>(a, r, blocks, s) : launch_one<8, 2, false>(a, r, blocks, s))
                             : (a.zp_u4 ? launch_one<8, 1, true>(a, r, blocks, s) : launch_one<8, 1, false>(a, r, blocks, s));
      }
      if (st) return st;
    }
    return 0;
  }
  // Everything else: the element-wise kernel on plain quantised activations,
  // in passes of as many rows as 64 MiB of scratch memory hold (the passes
  // follow one another on the stream, so they can share the buffer).
  const size_t row_bytes = (size_t)K * 2 + 2 * (size_t)a.G * sizeof(float) + 32;
  int64_t pass_rows = (int64_t)(((size_t)64 << 20) / row_bytes);
  if (pass_rows < 1) pass_rows = 1;
  if (pass_rows > M) pass_rows = M;
  const size_t q_bytes = ((size_t)pass_rows * K * 2 + 15) & ~(size_t)15;
  const size_t t_bytes = (size_t)pass_rows * a.G * sizeof(float);
  CallScratch lease(s, q_bytes + 2 * t_bytes);
  if (lease.overflowed()) return scratch_overflow_status("dequant_matmul_i4: the quantised activations", q_bytes + 2 * t_bytes);
  if (!lease.ptr()) return fail(8 /* RESOURCE_EXHAUSTED */, "dequant_matmul_i4: no scratch memory for the quantised activations");
  note_kernel_path("dequant_i4:reassociated-element-wise");
  ReassocArgs r = {};
  r.q_plain = (int16_t*)lease.ptr();
  r.scale_plain = (float*)((char*)lease.ptr() + q_bytes);
  r.sum_plain = r.scale_plain + (size_t)pass_rows * a.G;
  for (int64_t m0 = 0; m0 < M; m0 += pass_rows) {
    const int rows = (int)(M - m0 < pass_rows ? M - m0 : pass_rows);
    I4Args ap = a;
    ap.x = a.x + (size_t)m0 * K;
    ap.out = a.out + (size_t)m0 * N;
    ap.M = rows;
    hipLaunchKernelGGL(quantize_groups_i16_kernel, dim3(quantize_blocks(rows, a.G)), dim3(256), 0, s, ap.x, rows,
                       a.K, a.G, (int)group_size, 0, rows, r);
    UK_RETURN_IF_HIP(hipGetLastError());
    const int64_t total = (int64_t)rows * N;
    int64_t blocks = ceil_div(total, 256);
    const int64_t max_blocks = (int64_t)cus * 32;
    if (blocks > max_blocks) blocks = max_blocks;
    hipLaunchKernelGGL(dequant_matmul_i4_reassoc_generic_kernel, dim3((unsigned)blocks), dim3(256), 0, s, ap, r,
                       (int)group_size);
    UK_RETURN_IF_HIP(hipGetLastError());
  }
  return 0;
}

}  // namespace uk
