// mmt4d with a 16-bit left-hand side (S16S16S32, S16S8S32, S16U4S32; reference
// runtime/src/iree/builtins/ukernel/mmt4d_tile_generic.c:11-51,108-142,
// exported_bits.h:29-41) on the int8 matrix cores, by digit planes.
//
// A 16-bit value is x = 256 h + l + 128 with h = x >> 8 and l = (x & 255) - 128,
// both int8. The left-hand side becomes a tiled int8 operand of 2 M + 1 outer
// rows: the M rows of h, the M rows of l, and one row of the constant 64; a
// 16-bit right-hand side likewise 2 N + 1 outer rows (an 8- or 4-bit one is
// copied, the 4-bit one widened). One s8 x s8 mmt4d multiplies them into a
// tiled int32 product P in scratch memory, and a last pass adds the digit
// products with their weights:
//
//   8-bit rhs:  out = 256 P[h] + P[l] + 2 P[64]               (128 sum y = 2 * 64 sum y)
//   16-bit rhs: out = 65536 P[h,h] + 256 (P[h,l] + P[l,h]) + P[l,l]
//                     + 512 P[h,64] + 2 P[l,64] + 512 P[64,h] + 2 P[64,l] + 4 P[64,64]
//
// All of it is arithmetic modulo 2^32, like the reference's int32 accumulators,
// so the results are those of the element-wise kernel bit for bit. The planes
// are re-tiled to K0 = 16 on the way (any K0 of the call; the K positions past
// the end of a ragged K are zero in every plane, the constant one included), so
// the matrix-core kernel always sees its preferred tile.
//
// Narrow left-hand side tiles (one outer row of 1..15 rows against an 8- or
// 4-bit right-hand side: the reference's own s16 x u4 tile is 1 x 32 x 8,
// arch/x86_64/mmt4d_x86_64_tiles.inl:75) take the same route through the narrow
// matrix-core kernel: the planes are the 2 M0 + 1 rows of one int8 tile. With
// 16 to 31 rows those rows do not fit one narrow tile, and a 16-bit right-hand
// side has planes of its own: such tiles (one outer row) run as 32-row planes
// whose rows past M0 are zeros, the last pass storing M0 rows per tile.
#include "uk_common.h"

namespace uk {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

enum SourceKind { kSourceS16 = 0, kSourceS8 = 1, kSourceU4 = 2 };

struct RetileArgs {
  const void* src;        // element 0 of the buffer (offsets are in elements)
  int64_t offset, stride0;
  int64_t outer, K;       // outer rows and K tiles of the source
  int K0;
  int64_t k16;            // K tiles of the result: ceil(K * K0 / 16)
  uint8_t* dst;           // outer rows of k16 tiles of 32 x 16 bytes
  int src_rows;           // rows of a source tile: 32, or fewer (the result's rows beyond them are zeros)
};

// One thread makes row r of result tile (o, t): 16 consecutive K positions of
// source row 32 o + r. A 16-bit source writes its two digit planes (outer rows o
// and outer + o) and, from the threads of o = 0, the constant row 2 outer.
template <int kKind>
__global__ __launch_bounds__(256) void retile_planes_kernel(const RetileArgs a) {
  const int64_t total = a.outer * a.k16 * 32;
  const int64_t kk0 = a.K * a.K0;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int r = (int)(idx & 31);
    const int64_t t = (idx >> 5) % a.k16, o = (idx >> 5) / a.k16;
    const int64_t k_first = t * 16;
    int64_t kt = k_first / a.K0;
    int k0 = (int)(k_first - kt * a.K0);
    const int64_t base = a.offset + o * a.stride0;
    uint32_t hi[4] = {0, 0, 0, 0}, lo[4] = {0, 0, 0, 0}, cst[4] = {0, 0, 0, 0};
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      if (k_first + e < kk0 && r < a.src_rows) {
        const int64_t i = base + (kt * a.src_rows + r) * a.K0 + k0;
        const int sh = 8 * (e & 3);
        if (kKind == kSourceS16) {
          const int v = ((const int16_t*)a.src)[i];
          hi[e >> 2] |= (uint32_t)((v >> 8) & 255) << sh;
          lo[e >> 2] |= (uint32_t)(((v & 255) - 128) & 255) << sh;
          cst[e >> 2] |= 64u << sh;       // (row 0 is the one the last pass reads; it always exists)
        } else if (kKind == kSourceS8) {
          hi[e >> 2] |= (uint32_t)((const uint8_t*)a.src)[i] << sh;
        } else {
          const uint8_t b = ((const uint8_t*)a.src)[i >> 1];
          hi[e >> 2] |= (uint32_t)((i & 1) ? (b >> 4) : (b & 15)) << sh;
        }
      }
      if (++k0 == a.K0) { k0 = 0; ++kt; }
    }
    uint8_t* d = a.dst + ((o * a.k16 + t) * 32 + r) * 16;
    *(u32x4*)d = u32x4{hi[0], hi[1], hi[2], hi[3]};
    if (kKind == kSourceS16) {
      const int64_t plane = a.outer * a.k16 * 512;
      *(u32x4*)(d + plane) = u32x4{lo[0], lo[1], lo[2], lo[3]};
      if (o == 0) *(u32x4*)(d + 2 * plane) = u32x4{cst[0], cst[1], cst[2], cst[3]};
    }
  }
}

// The same for a 16-bit source whose K0 is a multiple of 8 and whose rows of 8
// elements are 16-byte aligned, with K * K0 whole 16-wide tiles: a thread's 16
// positions are two runs of 8 consecutive elements, loaded 16 bytes at a time;
// the high bytes of 4 elements are gathered with one byte permute, the low ones
// likewise and moved by 128 with an XOR ((b - 128) mod 256 = b ^ 0x80).
__global__ __launch_bounds__(256) void retile_planes_s16_wide_kernel(const RetileArgs a) {
  const int64_t total = a.outer * a.k16 * 32;
  const int64_t plane = a.outer * a.k16 * 512;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int r = (int)(idx & 31);
    const int64_t t = (idx >> 5) % a.k16, o = (idx >> 5) / a.k16;
    const int64_t base = a.offset + o * a.stride0;
    uint32_t hi[4], lo[4];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int64_t k = t * 16 + j * 8, kt = k / a.K0;
      const int k0 = (int)(k - kt * a.K0);
      const u32x4 v = *(const u32x4*)((const int16_t*)a.src + base + (kt * 32 + r) * a.K0 + k0);
      hi[2 * j] = __builtin_amdgcn_perm(v.y, v.x, 0x07050301u);
      hi[2 * j + 1] = __builtin_amdgcn_perm(v.w, v.z, 0x07050301u);
      lo[2 * j] = __builtin_amdgcn_perm(v.y, v.x, 0x06040200u) ^ 0x80808080u;
      lo[2 * j + 1] = __builtin_amdgcn_perm(v.w, v.z, 0x06040200u) ^ 0x80808080u;
    }
    uint8_t* d = a.dst + ((o * a.k16 + t) * 32 + r) * 16;
    *(u32x4*)d = u32x4{hi[0], hi[1], hi[2], hi[3]};
    *(u32x4*)(d + plane) = u32x4{lo[0], lo[1], lo[2], lo[3]};
    if (o == 0) *(u32x4*)(d + 2 * plane) = u32x4{0x40404040u, 0x40404040u, 0x40404040u, 0x40404040u};
  }
}

// The 4-bit right-hand side in tiles of K0 = 8 (the reference's s16 x u4 tile):
// a tile row is one dword of 8 nibbles, and rows r of two consecutive K tiles
// make one 16-byte row of the int8 tile. One thread per such row: two dword
// loads, the nibbles spread over bytes with two ANDs and two byte permutes
// each, one 16-byte store.
__global__ __launch_bounds__(256) void retile_u4_k8_kernel(const RetileArgs a) {
  const int64_t total = a.outer * a.k16 * 32;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int r = (int)(idx & 31);
    const int64_t t = (idx >> 5) % a.k16, o = (idx >> 5) / a.k16;
    const uint32_t* row = (const uint32_t*)((const uint8_t*)a.src + (a.offset + o * a.stride0) / 2) + (2 * t * 32 + r);
    const uint32_t w0 = 2 * t < a.K ? row[0] : 0u, w1 = 2 * t + 1 < a.K ? row[32] : 0u;
    const uint32_t lo0 = w0 & 0x0F0F0F0Fu, hi0 = (w0 >> 4) & 0x0F0F0F0Fu;
    const uint32_t lo1 = w1 & 0x0F0F0F0Fu, hi1 = (w1 >> 4) & 0x0F0F0F0Fu;
    *(u32x4*)(a.dst + idx * 16) = u32x4{__builtin_amdgcn_perm(hi0, lo0, 0x05010400u), __builtin_amdgcn_perm(hi0, lo0, 0x07030602u),
                                        __builtin_amdgcn_perm(hi1, lo1, 0x05010400u), __builtin_amdgcn_perm(hi1, lo1, 0x07030602u)};
  }
}

struct CombineArgs {
  const uint32_t* product;   // (2 M + 1) x cols tiles of 32 x 32
  int64_t M, N, cols;        // cols = N (narrow rhs) or 2 N + 1
  uint32_t* out;             // offset applied
  int64_t out_stride0;
  int accumulate;
  int rows;                  // rows of a result tile: 32, or the M0 of a narrow left-hand side
};

// One thread: 4 consecutive columns of one row of one result tile.
template <bool kWideRhs>
__global__ __launch_bounds__(256) void combine_planes_kernel(const CombineArgs a) {
  const int64_t total = a.M * a.N * 256;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int in_tile = (int)(idx & 255);            // row * 8 + group of 4 columns
    const int r = in_tile >> 3, c = (in_tile & 7) * 4;
    if (r >= a.rows) continue;
    const int64_t j = (idx >> 8) % a.N, i = (idx >> 8) / a.N;
    auto tile = [&](int64_t ti, int64_t tj) { return a.product + (ti * a.cols + tj) * 1024; };
    auto four = [&](const uint32_t* t, int row) { return *(const u32x4*)(t + row * 32 + c); };
    u32x4 v;
    if (!kWideRhs) {
      v = four(tile(i, j), r) * 256u + four(tile(a.M + i, j), r) + four(tile(2 * a.M, j), 0) * 2u;
    } else {
      const int64_t cj = 2 * a.N;                    // the constant column
      v = four(tile(i, j), r) * 65536u + (four(tile(i, a.N + j), r) + four(tile(a.M + i, j), r)) * 256u +
          four(tile(a.M + i, a.N + j), r) + four(tile(2 * a.M, j), 0) * 512u +
          four(tile(2 * a.M, a.N + j), 0) * 2u;
      v += tile(i, cj)[r * 32] * 512u + tile(a.M + i, cj)[r * 32] * 2u + tile(2 * a.M, cj)[0] * 4u;
    }
    uint32_t* o = a.out + i * a.out_stride0 + j * (a.rows * 32) + r * 32 + c;
    // (the result buffer is only element-aligned)
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = a.accumulate ? o[e] + v[e] : v[e];
  }
}

// Narrow left-hand side tiles (M0 < 16 rows, one outer row: the reference's own
// s16 x u4 tile is 1 x 32 x 8): the digit planes become the ROWS of one int8
// tile of 2 M0 + 1 rows (h rows, l rows, the constant row), which the narrow
// matrix-core kernel takes as it is.
struct RetileNarrowArgs {
  const int16_t* src;     // element 0 of the buffer
  int64_t offset;         // of the single outer row
  int64_t K;
  int K0, M0;
  int64_t k16;
  uint8_t* dst;           // k16 tiles of (2 M0 + 1) rows x 16 bytes
};

__global__ __launch_bounds__(256) void retile_planes_narrow_kernel(const RetileNarrowArgs a) {
  const int rows = 2 * a.M0 + 1;
  const int64_t total = a.k16 * rows;
  const int64_t kk0 = a.K * a.K0;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int r = (int)(idx % rows);
    const int64_t t = idx / rows;
    const int src_row = r < a.M0 ? r : r - a.M0;       // (unused for the constant row)
    int64_t kt = (t * 16) / a.K0;
    int k0 = (int)(t * 16 - kt * a.K0);
    uint32_t out[4] = {0, 0, 0, 0};
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      if (t * 16 + e < kk0) {
        uint32_t byte;
        if (r == 2 * a.M0) {
          byte = 64;
        } else {
          const int v = a.src[a.offset + (kt * a.M0 + src_row) * a.K0 + k0];
          byte = r < a.M0 ? (uint32_t)((v >> 8) & 255) : (uint32_t)(((v & 255) - 128) & 255);
        }
        out[e >> 2] |= byte << (8 * (e & 3));
      }
      if (++k0 == a.K0) { k0 = 0; ++kt; }
    }
    *(u32x4*)(a.dst + idx * 16) = u32x4{out[0], out[1], out[2], out[3]};
  }
}

struct CombineNarrowArgs {
  const uint32_t* product;   // N tiles of (2 M0 + 1) x 32
  int64_t N;
  int M0;
  uint32_t* out;             // N tiles of M0 x 32, offset applied
  int accumulate;
};

__global__ __launch_bounds__(256) void combine_planes_narrow_kernel(const CombineNarrowArgs a) {
  const int64_t total = a.N * a.M0 * 32;
  const int rows = 2 * a.M0 + 1;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int c = (int)(idx & 31);
    const int r = (int)((idx >> 5) % a.M0);
    const int64_t j = (idx >> 5) / a.M0;
    const uint32_t* t = a.product + j * rows * 32 + c;
    const uint32_t v = t[r * 32] * 256u + t[(a.M0 + r) * 32] + t[2 * a.M0 * 32] * 2u;
    a.out[idx] = a.accumulate ? a.out[idx] + v : v;
  }
}

template <typename Kernel, typename Args>
int launch_grid_stride(Kernel kernel, const Args& args, int64_t threads, hipStream_t s, const char* what);

// The 4-bit right-hand side as int8 tiles of K0 = 16.
int widen_u4_rhs(const RetileArgs& ra, hipStream_t s) {
  const bool dwords = ra.K0 == 8 && ra.offset % 8 == 0 && ra.stride0 % 8 == 0 && (uintptr_t)ra.src % 4 == 0;
  if (dwords) return launch_grid_stride(retile_u4_k8_kernel, ra, ra.outer * ra.k16 * 32, s, "mmt4d 4-bit rhs widening launch");
  return launch_grid_stride(retile_planes_kernel<kSourceU4>, ra, ra.outer * ra.k16 * 32, s, "mmt4d 4-bit rhs widening launch");
}

template <typename Kernel, typename Args>
int launch_grid_stride(Kernel kernel, const Args& args, int64_t threads, hipStream_t s, const char* what) {
  int64_t blocks = ceil_div(threads, (int64_t)256);
  const int64_t max_blocks = (int64_t)device_cu_count() * 32;
  if (blocks > max_blocks) blocks = max_blocks;
  hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(256), 0, s, args);
  return check_hip(hipGetLastError(), what);
}

inline size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

// Below this many multiply-accumulates the three extra launches cost more than
// the element-wise kernel takes.
constexpr int64_t kMinMacs = (int64_t)1 << 24;

}  // namespace

bool mmt4d_s16_planes_supported(uint32_t flags, int M0, int N0, int K0) {
  const uint32_t type = flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK;
  if (type != IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S16S32 && type != IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S8S32 &&
      type != IREE_AMD_UK_FLAG_MMT4D_TYPE_S16U4S32)
    return false;
  if (N0 != 32 || K0 < 1) return false;
  // 32 rows, and narrow left-hand sides of 1 to 31 (one outer row): up to 15
  // rows against an 8- or 4-bit right-hand side as the 2 M0 + 1 plane rows of
  // one narrow tile, the others as 32-row planes whose rows past M0 are zeros
  return M0 >= 1 && M0 <= 32 && mmt4d_mfma_supported(IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32, 32, 32, 16) &&
         mmt4d_skinny_supported(IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32, 31, 32, 16);
}

namespace {
int launch_narrow(const iree_amd_uk_mmt4d_params_t& p, hipStream_t s) {
  const uint32_t type = p.flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK;
  const int64_t kk0 = p.K * p.K0;
  if (p.M != 1 || p.K == 0 || (int64_t)p.M0 * 32 * p.N < ceil_div(kMinMacs / 2, kk0)) return IREE_AMD_UK_STATUS_NOT_FOUND;
  // (whole matrix-core steps of 32: the narrow kernel takes nothing else; the
  // positions past the end of K are zero in every plane)
  const int64_t k16 = 2 * ceil_div(kk0, (int64_t)32);
  const int rows = 2 * p.M0 + 1;
  const size_t lhs_bytes = align256((size_t)k16 * rows * 16), rhs_bytes = align256((size_t)p.N * k16 * 512);
  const size_t product_bytes = (size_t)p.N * rows * 32 * 4;
  ScratchLease lease(s, lhs_bytes + rhs_bytes + product_bytes);
  if (!lease.ptr()) return IREE_AMD_UK_STATUS_NOT_FOUND;
  uint8_t* lhs8 = (uint8_t*)lease.ptr();
  uint8_t* rhs8 = lhs8 + lhs_bytes;
  uint32_t* product = (uint32_t*)(rhs8 + rhs_bytes);
  const RetileNarrowArgs la = {(const int16_t*)p.lhs_buffer, p.lhs_offset, p.K, p.K0, p.M0, k16, lhs8};
  UK_RETURN_IF_ERROR(launch_grid_stride(retile_planes_narrow_kernel, la, k16 * rows, s,
                                        "mmt4d digit planes (narrow lhs) launch"));
  const RetileArgs ra = {p.rhs_buffer, p.rhs_offset, p.rhs_stride0, p.N, p.K, p.K0, k16, rhs8, 32};
  if (type == IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S8S32) {
    UK_RETURN_IF_ERROR(launch_grid_stride(retile_planes_kernel<kSourceS8>, ra, p.N * k16 * 32, s,
                                          "mmt4d 8-bit rhs re-tiling launch"));
  } else {
    UK_RETURN_IF_ERROR(widen_u4_rhs(ra, s));
  }
  iree_amd_uk_mmt4d_params_t q = {lhs8, 0, k16 * rows * 16, rhs8, 0, k16 * 512, product, 0, p.N * rows * 32,
                                  1, p.N, k16, rows, 32, 16, IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32, nullptr};
  {
    ScratchOverride none(nullptr, 0, /*strict=*/false);   // (the buffer is taken: no K split in there)
    UK_RETURN_IF_ERROR(iree_amd_uk_mmt4d_p(&q, s));
  }
  const CombineNarrowArgs ca = {product, p.N, p.M0, (uint32_t*)p.out_buffer + p.out_offset,
                                (p.flags & IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE) ? 1 : 0};
  return launch_grid_stride(combine_planes_narrow_kernel, ca, p.N * p.M0 * 32, s, "mmt4d digit combine launch");
}
}  // namespace

int launch_mmt4d_s16_planes(const iree_amd_uk_mmt4d_params_t& p, hipStream_t s) {
  if (!mmt4d_s16_planes_supported(p.flags, p.M0, p.N0, p.K0) || p.K == 0) return IREE_AMD_UK_STATUS_NOT_FOUND;
  const uint32_t type = p.flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK;
  const bool wide_rhs = type == IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S16S32;
  if (p.M0 != 32) {
    // narrow tiles exist for a single outer row only
    if (p.M != 1) return IREE_AMD_UK_STATUS_NOT_FOUND;
    if (!wide_rhs && p.M0 <= 15) return launch_narrow(p, s);
    // 16 to 31 rows (their 2 M0 + 1 plane rows do not fit one narrow tile),
    // and every narrow tile against a 16-bit right-hand side: the planes of
    // the 32-row form below, rows past M0 zero; the last pass stores M0 rows
  }
  const int64_t kk0 = p.K * p.K0;
  if (p.M * p.N * p.M0 * 32 < ceil_div(kMinMacs, kk0)) return IREE_AMD_UK_STATUS_NOT_FOUND;
  const int64_t k16 = ceil_div(kk0, (int64_t)16);
  const int64_t lhs_rows = 2 * p.M + 1, rhs_rows = wide_rhs ? 2 * p.N + 1 : p.N;
  if (lhs_rows > 0x7FFFFFFF / 64 || rhs_rows > 0x7FFFFFFF / 64) return IREE_AMD_UK_STATUS_NOT_FOUND;
  const size_t lhs_bytes = align256((size_t)lhs_rows * k16 * 512), rhs_bytes = align256((size_t)rhs_rows * k16 * 512);
  const size_t product_bytes = (size_t)lhs_rows * rhs_rows * 4096;
  const size_t bytes = lhs_bytes + rhs_bytes + product_bytes;
  ScratchLease lease(s, bytes);
  // (no memory, or a caller that brings too little of its own: the element-wise
  // kernel needs none)
  if (!lease.ptr()) return IREE_AMD_UK_STATUS_NOT_FOUND;
  uint8_t* lhs8 = (uint8_t*)lease.ptr();
  uint8_t* rhs8 = lhs8 + lhs_bytes;
  uint32_t* product = (uint32_t*)(rhs8 + rhs_bytes);

  // whole 16-byte runs of a 16-bit operand, 16-byte aligned, no ragged last tile
  auto wide = [&](const void* buffer, int64_t offset, int64_t stride0) {
    return p.K0 % 8 == 0 && kk0 % 16 == 0 && offset % 8 == 0 && stride0 % 8 == 0 && (uintptr_t)buffer % 16 == 0;
  };
  const RetileArgs la = {p.lhs_buffer, p.lhs_offset, p.lhs_stride0, p.M, p.K, p.K0, k16, lhs8, p.M0};
  if (p.M0 == 32 && wide(p.lhs_buffer, p.lhs_offset, p.lhs_stride0)) {
    UK_RETURN_IF_ERROR(launch_grid_stride(retile_planes_s16_wide_kernel, la, p.M * k16 * 32, s,
                                          "mmt4d digit planes (lhs) launch"));
  } else {
    UK_RETURN_IF_ERROR(launch_grid_stride(retile_planes_kernel<kSourceS16>, la, p.M * k16 * 32, s,
                                          "mmt4d digit planes (lhs) launch"));
  }
  const RetileArgs ra = {p.rhs_buffer, p.rhs_offset, p.rhs_stride0, p.N, p.K, p.K0, k16, rhs8, 32};
  const uint8_t* rhs_operand = rhs8;
  int64_t rhs_operand_stride = k16 * 512;
  if (wide_rhs) {
    if (wide(p.rhs_buffer, p.rhs_offset, p.rhs_stride0)) {
      UK_RETURN_IF_ERROR(launch_grid_stride(retile_planes_s16_wide_kernel, ra, p.N * k16 * 32, s,
                                            "mmt4d digit planes (rhs) launch"));
    } else {
      UK_RETURN_IF_ERROR(launch_grid_stride(retile_planes_kernel<kSourceS16>, ra, p.N * k16 * 32, s,
                                            "mmt4d digit planes (rhs) launch"));
    }
  } else if (type == IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S8S32 && p.K0 == 16 && p.rhs_offset % 16 == 0 &&
             p.rhs_stride0 % 16 == 0 && (uintptr_t)p.rhs_buffer % 16 == 0) {
    // (already what the matrix-core kernel takes: used where it lies)
    rhs_operand = (const uint8_t*)p.rhs_buffer + p.rhs_offset;
    rhs_operand_stride = p.rhs_stride0;
  } else if (type == IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S8S32) {
    UK_RETURN_IF_ERROR(launch_grid_stride(retile_planes_kernel<kSourceS8>, ra, p.N * k16 * 32, s,
                                          "mmt4d 8-bit rhs re-tiling launch"));
  } else {
    UK_RETURN_IF_ERROR(widen_u4_rhs(ra, s));
  }

  iree_amd_uk_mmt4d_params_t q = {lhs8, 0, k16 * 512, rhs_operand, 0, rhs_operand_stride, product, 0, rhs_rows * 1024,
                                  lhs_rows, rhs_rows, k16, 32, 32, 16, IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32,
                                  nullptr};
  {
    // The stream's scratch buffer holds the operands and the product: the
    // matmul itself runs without scratch memory (no K split).
    ScratchOverride none(nullptr, 0, /*strict=*/false);
    UK_RETURN_IF_ERROR(iree_amd_uk_mmt4d_p(&q, s));
  }
  const CombineArgs ca = {product, p.M, p.N, rhs_rows, (uint32_t*)p.out_buffer + p.out_offset, p.out_stride0,
                          (p.flags & IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE) ? 1 : 0, p.M0};
  if (wide_rhs)
    return launch_grid_stride(combine_planes_kernel<true>, ca, p.M * p.N * 256, s, "mmt4d digit combine launch");
  return launch_grid_stride(combine_planes_kernel<false>, ca, p.M * p.N * 256, s, "mmt4d digit combine launch");
}

}  // namespace uk
