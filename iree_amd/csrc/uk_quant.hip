// Grouped int4-weight dequantising matmul and the fp8 element-wise helpers.
//
//   out[m][n] = sum_g s[n][g] * sum_{k in g} x[m][k] * (w[n][k] - zp[n][g])
//
// (the fused dequantisation + matmul pattern of the reference's
// compiler/src/iree/compiler/GlobalOptimization/FuseDequantizationMatmul.cpp:53-159;
// f32 accumulation, one rounding to f16 at the end).
//
// Decode-shaped calls (a few rows of activations) are bound by the HBM stream of
// the weights, 0.5 byte per weight, and the whole stream is only tens of
// megabytes: the kernel is as much latency- as bandwidth-bound. The fast kernel
// therefore:
//   * reads each weight byte exactly once, 16 bytes per lane per load, through
//     buffer loads that always have a whole tile of requests in flight: the
//     request for slab i of the next tile is issued the moment slab i of the
//     current tile has been consumed, and nothing in the loop waits for a load
//     it has just issued (group parameters travel as raw bits and are only
//     decoded when the weights that follow them in the queue have landed);
//   * keeps the activations stationary in REGISTERS: the 8 waves of a
//     workgroup each own one eighth of K and hold their slice of x as MFMA A
//     operands for the whole kernel, so no LDS or cache bandwidth is spent on
//     re-reading x (which would be 4 bytes per weight byte); LDS only stages
//     them once on the way in;
//   * dequantises in registers ahead of the MFMA with as few vector
//     instructions as the format allows, because the tile loop is bound by
//     them: the nibbles go to v_mfma_f32_16x16x32_f16 as f16 subnormals (one
//     shift and four ANDs per 8 weights, every product exact in f32), the zero
//     point is applied through per-group sums of the activations that the
//     matrix cores take once per workgroup, and the per-group f32 partial sums
//     are scaled by s[n][g] with one f32 FMA per accumulator register (the lane
//     owns column n, so scale and zero point are per-lane scalars). Instances
//     without register room for the group sums turn a nibble n into the f16
//     value 1024+n (or 1024+16n for the upper nibble of a byte) by OR-ing it
//     into the mantissa of 0x6400 and remove offset and zero point with exact
//     packed-f16 arithmetic;
//   * sums the 8 K-slices through LDS in a fixed order (deterministic).
#include "uk_common.h"
#include "uk_fp8.h"
#include "uk_i4.h"
#include "uk_i4_kernel.h"

#include <memory>

#include <hip/hip_fp16.h>

namespace uk {
using namespace i4;
namespace {

template <int KB, int MH, bool kZpU4, int kLog2Gs>
__global__ __launch_bounds__(kThreads) void dequant_matmul_i4_kernel(I4Args a) {
  dequant_matmul_i4_body<KB, MH, kZpU4, kLog2Gs>(a);
}

// Row-major [N][K/2] bytes -> the tiled layout (one thread per dword).
__global__ __launch_bounds__(256) void pack_i4_weights_kernel(const uint32_t* src, uint32_t* dst,
                                                              int64_t N, int64_t K) {
  const int64_t total = N * K / 8;
  for (int64_t d = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; d < total;
       d += (int64_t)gridDim.x * blockDim.x) {
    const int64_t q = d & 3, kc = (d >> 2) & 3, c = (d >> 4) & 31, rest = d >> 9;
    const int64_t spans = K >> 7, s = rest % spans, nt = rest / spans;
    dst[d] = src[((nt * 32 + c) * K + s * 128 + q * 32 + kc * 8) >> 3];
  }
}

// Reference-order fallback for every shape the MFMA kernel does not serve: one
// thread per output element.
__global__ __launch_bounds__(256) void dequant_matmul_i4_generic_kernel(I4Args a, int gs) {
  const int64_t total = (int64_t)a.M * a.N;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int m = (int)(idx / a.N), n = (int)(idx - (int64_t)m * a.N);
    float acc = 0.f;
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
      float part = 0.f;
      for (int kk = 0; kk < gs; ++kk) {
        const int k = g * gs + kk;
        const uint8_t byte = a.w[a.tiled ? tiled_byte_index(n, k, a.K) : ((size_t)n * a.K + k) >> 1];
        const float q = (float)((k & 1) ? (byte >> 4) : (byte & 0xF));
        part = __builtin_fmaf(__half2float(__ushort_as_half(a.x[(size_t)m * a.K + k])), q - zpv, part);
      }
      acc = __builtin_fmaf(part, sc, acc);
    }
    a.out[idx] = __half_as_ushort(__float2half_rn(acc));
  }
}

template <int KB, int MH, bool kZpU4, int kLog2Gs>
int launch_instance(const I4Args& a, int blocks, int k_rows, hipStream_t s) {
  void (*kernel)(I4Args) = dequant_matmul_i4_kernel<KB, MH, kZpU4, kLog2Gs>;
  // 16-row form: the rows it stages (8 or 16 per wave); 32-row form: two
  // buffers of one span (128 k of 32 rows) per wave, and at least the 64 KiB of
  // partial sums that later live in the same memory
  constexpr size_t kMaxLds = MH == 2 ? (size_t)kWaves * 2 * 32 * 256    // two spans of 32 rows per wave
                                     : (size_t)kWaves * kStageRowsMax * stage_row_bytes<KB>();
  constexpr size_t kPartialBytes = MH == 2 ? (size_t)2 * kWaves * 2 * MH * 4 * 64 * sizeof(float) : 0;
  constexpr size_t kAttrLds = kMaxLds > kPartialBytes ? kMaxLds : kPartialBytes;
  const size_t lds = MH == 1 ? (size_t)kWaves * a.stage_rows * stage_row_bytes<KB>() : kAttrLds;
  {
    // (with the 16-row form's static 32 KiB this is more than the 64 KiB a kernel gets by default)
    static PerDeviceOnce attr_set_on;
    int dev = 0;
    UK_RETURN_IF_HIP(hipGetDevice(&dev));
    if (!attr_set_on.done(dev)) {
      UK_RETURN_IF_HIP(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)kAttrLds));
      attr_set_on.mark(dev);
    }
  }
  hipLaunchKernelGGL(kernel, dim3(blocks, k_rows), dim3(kThreads), lds, s, a);
  return check_hip(hipGetLastError(), "dequant_matmul_i4 launch");
}

template <int KB, int MH, bool kZpU4>
int launch_one(const I4Args& a, int blocks, int k_rows, hipStream_t s) {
  // (with K rows a group may be longer than a workgroup's slice of K: it is
  // then "at least the wave's slice" all the same)
  switch (a.log2_gs) {
    case 5: return launch_instance<KB, MH, kZpU4, 5>(a, blocks, k_rows, s);
    case 6: return launch_instance<KB, MH, kZpU4, 6>(a, blocks, k_rows, s);
    case 7: return launch_instance<KB, MH, kZpU4, 7>(a, blocks, k_rows, s);
    case 8: return launch_instance<KB, MH, kZpU4, 8>(a, blocks, k_rows, s);
    default: return launch_instance<KB, MH, kZpU4, 9>(a, blocks, k_rows, s);
  }
}

// K = k_rows slices of 512 KB elements. One slice: f16 results straight to the
// output. More: every workgroup row multiplies its slice into f32 partial sums
// in the stream's scratch buffer and the K-split reduction kernel adds them in
// row order and rounds to f16 once (NOT_FOUND without that memory: the caller
// falls back to the kernel that walks all of K in one workgroup).
template <int KB>
int launch_fast(I4Args a, int k_rows, hipStream_t s) {
  const int cus = device_cu_count();
  std::unique_ptr<ScratchLease> lease;   // held until the reduction has been queued
  a.partial = nullptr;
  if (k_rows > 1) {
    if (((int64_t)a.M * a.N) % 4) return IREE_AMD_UK_STATUS_NOT_FOUND;
    lease.reset(new ScratchLease(s, (size_t)k_rows * a.M * a.N * 4));
    a.partial = (float*)lease->ptr();
    if (!a.partial) return IREE_AMD_UK_STATUS_NOT_FOUND;
  }
  int m_base = 0;
  while (m_base < a.M) {
    a.m_base = m_base;
    // One workgroup per compute unit (two of the 16-row kernel would fit, and
    // measure slower: 12.4 against 9.9 us on the decode shape); with K rows,
    // a row gets its share of the compute units.
    int blocks = cus / k_rows;
    blocks = blocks < 1 ? 1 : blocks;
    blocks = a.n_tiles < blocks ? a.n_tiles : blocks;
    int st;
    if (a.M - m_base > 16) {
      st = a.zp_u4 ? launch_one<KB, 2, true>(a, blocks, k_rows, s) : launch_one<KB, 2, false>(a, blocks, k_rows, s);
      m_base += 32;
    } else {
      a.stage_rows = stage_rows_for(a.M - m_base);
      st = a.zp_u4 ? launch_one<KB, 1, true>(a, blocks, k_rows, s) : launch_one<KB, 1, false>(a, blocks, k_rows, s);
      m_base += 16;
    }
    UK_RETURN_IF_ERROR(st);
  }
  if (k_rows == 1) return 0;
  KSplitReduceArgs r;
  r.partials = a.partial;
  r.slices = k_rows;
  r.M = 1; r.N = 1;
  r.flat_elems = (int64_t)a.M * a.N;
  r.out = a.out;
  r.out_stride_bytes = 0;
  r.accumulate = 0;
  r.row_major_out = 0; r.out_rows = r.out_cols = 0;
  r.out_scale = 1.0f;
  r.acc_is_float = 1;
  r.out_kind = 1;   // f16
  return launch_ksplit_reduce(r, s);
}

}  // namespace

int launch_dequant_matmul_i4(const void* x, const void* w, const void* scale, const void* zp,
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
  a.span_stride = tiled ? 2048u : 64u;
  a.col_stride = tiled ? 64u : (uint32_t)(K / 2);
  // Fast path: K in slices of 512 * KB for KB in {4, 8} (every wave owns
  // KB blocks of 64 of its workgroup's slice; more than one slice: workgroup
  // rows and a second kernel that adds their partial sums; K in whole 256s,
  // the last slice as short as that leaves it),
  // power-of-two groups (below 128 only from tiled weights, where a group never
  // straddles an MFMA), a weight buffer that 32-bit offsets can address (plus
  // one tile, for the offset of the tile after the last), 16-byte aligned
  // operands, and group parameters aligned to what one wave slice loads at once.
  const int64_t w_bytes = N * K / 2;
  // (a longer K in whole slices of 4096, or else of 2048, over workgroup rows)
  // (any other K in whole wave slices of 256: slices of 2048 whose last one is
  // shorter, its trailing waves running on zeros)
  const int slice_kb = K % 4096 == 0 ? 8 : 4;
  const int64_t k_rows = ceil_div(K, (int64_t)512 * slice_kb);
  const bool k_ok = K % 256 == 0 && K >= 256 && k_rows <= 64 && (group_size <= 256 || K % 2048 == 0);
  const bool gs_ok = gs_pow2 && group_size >= (tiled ? 32 : 128);
  const bool size_ok = w_bytes + K * 16 < (1ll << 32);
  const bool aligned = ((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0 &&
                       ((uintptr_t)scale % 16) == 0 && ((uintptr_t)zp % 16) == 0;
  // (one row against few tiles of columns and a split K: the kernel below, in
  // which a wave walks all of K for its columns, measures a little faster, 11.1
  // against 11.9 us at N = 4096, K = 14336, and needs no second launch)
  const bool one_row_few_tiles = M == 1 && k_rows > 1 && a.n_tiles * 2 <= device_cu_count() && K % 2048 == 0 &&
                                 group_size >= (tiled ? 64 : 128) && group_size <= 256;
  if (k_ok && gs_ok && size_ok && aligned && !one_row_few_tiles) {
    a.w_bytes = (uint32_t)w_bytes;
    const int st = slice_kb == 4 ? launch_fast<4>(a, (int)k_rows, s) : launch_fast<8>(a, (int)k_rows, s);
    if (st != IREE_AMD_UK_STATUS_NOT_FOUND) { note_kernel_path("dequant_i4:mfma"); return st; }
  }
  if (gs_pow2 && size_ok && aligned && K > 0) {
    // Other K (whole 2048s): the per-wave-column kernel. It has a longer
    // start-up (one wave walks all of K for its columns) but no limit on K as
    // long as one row of activations fits LDS. Rows go in passes of as many
    // as fit (at most 16), each pass streaming the weights again: up to 8
    // passes are still far cheaper than the element-wise kernel.
    a.w_bytes = (uint32_t)w_bytes;
    // First with 16 rows per pass whatever K is (the kernel splits a K whose
    // activations do not fit LDS over workgroup rows, which needs scratch
    // memory), then with as many rows as fit without that.
    for (int attempt = 0; attempt < 2; ++attempt) {
      int64_t rows_per_pass = attempt == 0 ? 16 : (144 * 1024) / (K * 2);
      if (rows_per_pass > 16) rows_per_pass = 16;
      if (rows_per_pass < 1 || ceil_div(M, rows_per_pass) > 8) continue;
      // equal passes (8 rows at 5 per pass: 4 + 4 rather than 5 + 3)
      const int64_t passes = ceil_div(M, rows_per_pass);
      const int64_t rows = ceil_div(M, passes);
      int st = 0;
      for (int64_t m0 = 0; m0 < M; m0 += rows) {
        st = launch_dequant_gemv_i4(a, (int)m0, (int)(M - m0 < rows ? M - m0 : rows), s);
        if (st) break;     // NOT_FOUND can only come from the first pass: nothing has run yet
      }
      if (st != IREE_AMD_UK_STATUS_NOT_FOUND) { note_kernel_path("dequant_i4:gemv"); return st; }
    }
  }
  if (one_row_few_tiles && k_ok && gs_ok && size_ok && aligned) {
    a.w_bytes = (uint32_t)w_bytes;
    const int st = slice_kb == 4 ? launch_fast<4>(a, (int)k_rows, s) : launch_fast<8>(a, (int)k_rows, s);
    if (st != IREE_AMD_UK_STATUS_NOT_FOUND) { note_kernel_path("dequant_i4:mfma"); return st; }
  }
  const int64_t total = M * N;
  int64_t blocks = ceil_div(total, 256);
  const int64_t max_blocks = (int64_t)device_cu_count() * 32;
  if (blocks > max_blocks) blocks = max_blocks;
  note_kernel_path("dequant_i4:element-wise");
  hipLaunchKernelGGL(dequant_matmul_i4_generic_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a,
                     (int)group_size);
  return check_hip(hipGetLastError(), "dequant_matmul_i4_generic launch");
}

int launch_pack_i4_weights(const void* src, void* dst, int64_t N, int64_t K, hipStream_t s) {
  const int64_t total = N * K / 8;
  if (total == 0) return 0;
  int64_t blocks = ceil_div(total, 256);
  const int64_t max_blocks = (int64_t)device_cu_count() * 32;
  if (blocks > max_blocks) blocks = max_blocks;
  hipLaunchKernelGGL(pack_i4_weights_kernel, dim3((unsigned)blocks), dim3(256), 0, s,
                     (const uint32_t*)src, (uint32_t*)dst, N, K);
  return check_hip(hipGetLastError(), "pack_i4_weights launch");
}

//===----------------------------------------------------------------------===//
// fp8 element-wise helpers of the MLP block. All of them are HBM streams:
// 16-byte accesses, no reuse.
//===----------------------------------------------------------------------===//

namespace {

__global__ __launch_bounds__(256) void quantize_f16_kernel(const uint16_t* in, uint8_t* out,
                                                           int64_t n, float inv_scale) {
  const int64_t n8 = n >> 3;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8;
       i += (int64_t)gridDim.x * blockDim.x) {
    const u32x4 v = ((const u32x4*)in)[i];
    float f[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f[2 * j] = __half2float(__ushort_as_half((uint16_t)(v[j] & 0xFFFF))) * inv_scale;
      f[2 * j + 1] = __half2float(__ushort_as_half((uint16_t)(v[j] >> 16))) * inv_scale;
    }
    ((u32x2*)out)[i] = u32x2{pack4_e4m3(f[0], f[1], f[2], f[3]), pack4_e4m3(f[4], f[5], f[6], f[7])};
  }
  // tail (n % 8 elements) and unaligned buffers: element-wise
  if (blockIdx.x == 0) {
    for (int64_t i = (n8 << 3) + threadIdx.x; i < n; i += blockDim.x) {
      const float f = __half2float(__ushort_as_half(in[i])) * inv_scale;
      out[i] = (uint8_t)(pack4_e4m3(f, 0.f, 0.f, 0.f) & 0xFF);
    }
  }
}

// Quantisation and the pack of the result in one pass: f16 row-major
// [rows][cols] -> e4m3 left-hand-side tiles [ceil(rows/32)][cols/16][32][16],
// rows past `rows` zero (the padding value of that pack). A lane makes one
// 16-byte tile row from 32 bytes of a matrix row; lane = (row in block) * 8 +
// (tile column in block) as in the streaming pack, so a wave reads 8 row
// pieces of 256 bytes and writes 8 runs of 128 bytes, and a workgroup's four
// waves complete 8 whole tiles.
typedef u32x4 u32x4_align2 __attribute__((aligned(2)));
__global__ __launch_bounds__(256) void quantize_pack_f8_kernel(const uint16_t* in, int64_t ld, uint8_t* out,
                                                               int64_t out_stride0, int64_t rows, int64_t k_tiles,
                                                               float inv_scale) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t kt = (int64_t)blockIdx.x * 8 + (lane & 7);
  const int row_in_tile = wave * 8 + (lane >> 3);
  const int64_t row = (int64_t)blockIdx.y * 32 + row_in_tile;
  if (kt >= k_tiles) return;
  u32x2 q0 = {0u, 0u}, q1 = {0u, 0u};
  if (row < rows) {
    const uint16_t* src = in + row * ld + kt * 16;
    const u32x4 a = *(const u32x4_align2*)src, b = *(const u32x4_align2*)(src + 8);
    float f[16];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f[2 * j] = __half2float(__ushort_as_half((uint16_t)(a[j] & 0xFFFF))) * inv_scale;
      f[2 * j + 1] = __half2float(__ushort_as_half((uint16_t)(a[j] >> 16))) * inv_scale;
      f[8 + 2 * j] = __half2float(__ushort_as_half((uint16_t)(b[j] & 0xFFFF))) * inv_scale;
      f[8 + 2 * j + 1] = __half2float(__ushort_as_half((uint16_t)(b[j] >> 16))) * inv_scale;
    }
    q0 = u32x2{pack4_e4m3(f[0], f[1], f[2], f[3]), pack4_e4m3(f[4], f[5], f[6], f[7])};
    q1 = u32x2{pack4_e4m3(f[8], f[9], f[10], f[11]), pack4_e4m3(f[12], f[13], f[14], f[15])};
  }
  uint8_t* dst = out + (int64_t)blockIdx.y * out_stride0 + kt * 512 + row_in_tile * 16;
  *(u32x4*)dst = u32x4{q0.x, q0.y, q1.x, q1.y};
}

__global__ __launch_bounds__(256) void quantize_f16_scalar_kernel(const uint16_t* in, uint8_t* out,
                                                                  int64_t n, float inv_scale) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const float f = __half2float(__ushort_as_half(in[i])) * inv_scale;
    out[i] = (uint8_t)(pack4_e4m3(f, 0.f, 0.f, 0.f) & 0xFF);
  }
}

// Row-major: thread = 4 consecutive columns of one row when everything is
// 16-byte aligned (kVec), else one element.
template <bool kVec>
__global__ __launch_bounds__(256) void silu_mul_quantize_kernel(const float* gate, const float* up,
                                                                uint8_t* out, int64_t rows,
                                                                int64_t cols, int64_t ld, float gs,
                                                                float us, float os) {
  constexpr int V = kVec ? 4 : 1;
  const int64_t per_row = cols / V, total = rows * per_row;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / per_row, c = (i - r * per_row) * V;
    if constexpr (kVec) {
      const floatx4 g = *(const floatx4*)(gate + r * ld + c), u = *(const floatx4*)(up + r * ld + c);
      float h[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) h[j] = silu_mul(g[j] * gs, u[j] * us) * os;
      *(uint32_t*)(out + r * cols + c) = pack4_e4m3(h[0], h[1], h[2], h[3]);
    } else {
      const float h = silu_mul(gate[r * ld + c] * gs, up[r * ld + c] * us) * os;
      out[r * cols + c] = (uint8_t)(pack4_e4m3(h, 0.f, 0.f, 0.f) & 0xFF);
    }
  }
}

// Tiled: one wave per pair (gate tile, up tile) of 32x32 f32 accumulators;
// lane l owns row l / 2, columns (l % 2) * 16 .. + 16: 64 contiguous bytes of
// each input tile and 16 contiguous bytes of the output, which is the pair of
// adjacent 32x16 e4m3 left-hand-side tiles (2j, 2j+1) of outer row i.
__global__ __launch_bounds__(256) void silu_mul_quantize_tiled_kernel(
    const float* acc, int64_t acc_stride0, int64_t gate_tile0, int64_t up_tile0, uint8_t* out,
    int64_t out_stride0, int64_t M1, int64_t N1, float gs, float us, float os) {
  const int lane = threadIdx.x & 63;
  const int64_t pair = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (pair >= M1 * N1) return;
  const int64_t i = pair / N1, j = pair - i * N1;
  const float* g = acc + i * acc_stride0 + (gate_tile0 + j) * 1024 + lane * 16;
  const float* u = acc + i * acc_stride0 + (up_tile0 + j) * 1024 + lane * 16;
  uint32_t w[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const floatx4 gv = ((const floatx4*)g)[q], uv = ((const floatx4*)u)[q];
    float h[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) h[e] = silu_mul(gv[e] * gs, uv[e] * us) * os;
    w[q] = pack4_e4m3(h[0], h[1], h[2], h[3]);
  }
  uint8_t* o = out + i * out_stride0 + j * 1024 + (lane & 1) * 512 + (lane >> 1) * 16;
  *(u32x4*)o = u32x4{w[0], w[1], w[2], w[3]};
}

template <bool kVec>
__global__ __launch_bounds__(256) void scale_f32_kernel(float* buf, int64_t n, float scale) {
  const int64_t n4 = kVec ? n >> 2 : 0;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4;
       i += (int64_t)gridDim.x * blockDim.x) {
    floatx4 v = ((floatx4*)buf)[i];
    v[0] *= scale; v[1] *= scale; v[2] *= scale; v[3] *= scale;
    ((floatx4*)buf)[i] = v;
  }
  for (int64_t i = (n4 << 2) + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x)
    buf[i] *= scale;
}

unsigned stream_blocks(int64_t work_items) {
  int64_t blocks = ceil_div(work_items, (int64_t)256);
  const int64_t max_blocks = (int64_t)device_cu_count() * 16;
  if (blocks > max_blocks) blocks = max_blocks;
  return (unsigned)(blocks < 1 ? 1 : blocks);
}

}  // namespace

int launch_quantize_f16_to_f8e4m3(const void* in, void* out, int64_t n, float inv_scale,
                                  hipStream_t s) {
  if (((uintptr_t)in % 16) == 0 && ((uintptr_t)out % 8) == 0) {
    hipLaunchKernelGGL(quantize_f16_kernel, dim3(stream_blocks(n / 8)), dim3(256), 0, s,
                       (const uint16_t*)in, (uint8_t*)out, n, inv_scale);
  } else {
    hipLaunchKernelGGL(quantize_f16_scalar_kernel, dim3(stream_blocks(n)), dim3(256), 0, s,
                       (const uint16_t*)in, (uint8_t*)out, n, inv_scale);
  }
  return check_hip(hipGetLastError(), "quantize_f16_to_f8e4m3 launch");
}

int launch_quantize_pack_f8e4m3(const void* in, int64_t ld, void* out, int64_t out_stride0, int64_t rows,
                                int64_t cols, float inv_scale, hipStream_t s) {
  const int64_t k_tiles = cols / 16, row_tiles = ceil_div(rows, 32);
  if (row_tiles > 65535 || ceil_div(k_tiles, 8) > 0x7FFFFFFF)
    return fail(IREE_AMD_UK_STATUS_UNIMPLEMENTED, "quantize_pack: more than 65535 outer rows");
  hipLaunchKernelGGL(quantize_pack_f8_kernel, dim3((unsigned)ceil_div(k_tiles, 8), (unsigned)row_tiles), dim3(256), 0, s,
                     (const uint16_t*)in, ld, (uint8_t*)out, out_stride0, rows, k_tiles, inv_scale);
  return check_hip(hipGetLastError(), "quantize_pack launch");
}

int launch_silu_mul_quantize(const void* gate, const void* up, void* out, int64_t rows,
                             int64_t cols, int64_t ld, float gate_scale, float up_scale,
                             float inv_out_scale, hipStream_t s) {
  const bool vec = cols % 4 == 0 && ld % 4 == 0 && ((uintptr_t)gate % 16) == 0 &&
                   ((uintptr_t)up % 16) == 0 && ((uintptr_t)out % 4) == 0;
  if (vec) {
    hipLaunchKernelGGL(silu_mul_quantize_kernel<true>, dim3(stream_blocks(rows * cols / 4)), dim3(256),
                       0, s, (const float*)gate, (const float*)up, (uint8_t*)out, rows, cols, ld,
                       gate_scale, up_scale, inv_out_scale);
  } else {
    hipLaunchKernelGGL(silu_mul_quantize_kernel<false>, dim3(stream_blocks(rows * cols)), dim3(256),
                       0, s, (const float*)gate, (const float*)up, (uint8_t*)out, rows, cols, ld,
                       gate_scale, up_scale, inv_out_scale);
  }
  return check_hip(hipGetLastError(), "silu_mul_quantize launch");
}

int launch_silu_mul_quantize_tiled(const void* acc, int64_t acc_stride0, int64_t gate_tile0,
                                   int64_t up_tile0, void* out, int64_t out_stride0, int64_t M1,
                                   int64_t N1, float gate_scale, float up_scale,
                                   float inv_out_scale, hipStream_t s) {
  const int64_t blocks = ceil_div(M1 * N1, (int64_t)4);
  if (blocks > 0x7FFFFFFF)
    return fail(IREE_AMD_UK_STATUS_OUT_OF_RANGE, "silu_mul_quantize_tiled: too many tiles");
  hipLaunchKernelGGL(silu_mul_quantize_tiled_kernel, dim3((unsigned)blocks), dim3(256), 0, s,
                     (const float*)acc, acc_stride0, gate_tile0, up_tile0, (uint8_t*)out,
                     out_stride0, M1, N1, gate_scale, up_scale, inv_out_scale);
  return check_hip(hipGetLastError(), "silu_mul_quantize_tiled launch");
}

int launch_scale_f32(void* buf, int64_t n, float scale, hipStream_t s) {
  if ((uintptr_t)buf % 16 == 0) {
    hipLaunchKernelGGL(scale_f32_kernel<true>, dim3(stream_blocks(n / 4)), dim3(256), 0, s,
                       (float*)buf, n, scale);
  } else {
    hipLaunchKernelGGL(scale_f32_kernel<false>, dim3(stream_blocks(n)), dim3(256), 0, s, (float*)buf,
                       n, scale);
  }
  return check_hip(hipGetLastError(), "scale_f32 launch");
}

}  // namespace uk
