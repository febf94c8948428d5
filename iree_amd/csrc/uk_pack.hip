// pack / unpack kernels.
//
// Semantics (runtime/src/iree/builtins/ukernel/tools/pack_test.c:13-71 and
// unpack_test.c:13-58 of the reference): a strided 2-D matrix <-> a 4-D array
// of tiles, with optional swaps of the two outer and of the two inner tile
// dimensions, and - for pack only - a padding element wherever a tile sticks
// out of the matrix.
//
// Two kernel families:
//   *_generic : one thread per destination element; every type, transpose,
//               stride and offset combination.
//   *_stream  : HBM-streaming path for the common layout (unit inner stride of
//               the matrix, no inner transpose, tile rows that are whole 16-byte
//               chunks, 16-byte aligned tiled buffer). Each lane moves one
//               16-byte chunk with a single 128-bit load and store; lanes are
//               laid out along the DESTINATION so every wave writes 1 KiB
//               contiguous, and each wave walks four neighbouring units that
//               share their source cache lines. Matrix rows need only element
//               alignment: the hardware performs the unaligned 128-bit
//               accesses.
#include "uk_common.h"

namespace uk {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// 128-bit access to memory that is only element-aligned.
template <int ES> struct Chunk;
template <> struct Chunk<1> { typedef u32x4 aligned_t __attribute__((aligned(1))); };
template <> struct Chunk<2> { typedef u32x4 aligned_t __attribute__((aligned(2))); };
template <> struct Chunk<4> { typedef u32x4 aligned_t __attribute__((aligned(4))); };

struct PackArgs {
  const char* in;   // matrix (pack source / unpack destination), offset applied
  char* out;        // tiled buffer, offset applied
  int64_t m_size0, m_size1, m_stride0, m_stride1;  // matrix, elements
  int64_t t_size0, t_size1;                         // tiled outer sizes as stored
  int64_t t_stride0;                                // elements
  int t_size2, t_size3;                             // tile sizes as stored
  int transpose_inner, transpose_outer;
  uint64_t padding;
};

template <typename T>
__device__ __forceinline__ T pad_value(uint64_t padding) {
  return (T)padding;
}

// One thread per element of the tiled buffer.
template <typename T>
__global__ __launch_bounds__(256) void pack_generic_kernel(PackArgs a) {
  const int64_t tile_elems = (int64_t)a.t_size2 * a.t_size3;
  const int64_t total = a.t_size0 * a.t_size1 * tile_elems;
  const T* in = (const T*)a.in;
  T* out = (T*)a.out;
  const T pad = pad_value<T>(a.padding);
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t tile = idx / tile_elems;
    const int e = (int)(idx - tile * tile_elems);
    const int64_t d0 = tile / a.t_size1, d1 = tile - d0 * a.t_size1;
    const int d2 = e / a.t_size3, d3 = e - d2 * a.t_size3;
    const int64_t orow = a.transpose_outer ? d1 : d0, ocol = a.transpose_outer ? d0 : d1;
    const int trow = a.transpose_inner ? d3 : d2, tcol = a.transpose_inner ? d2 : d3;
    const int tile_rows = a.transpose_inner ? a.t_size3 : a.t_size2;
    const int tile_cols = a.transpose_inner ? a.t_size2 : a.t_size3;
    const int64_t r = orow * tile_rows + trow, c = ocol * tile_cols + tcol;
    const int64_t dst = d0 * a.t_stride0 + d1 * tile_elems + e;
    out[dst] = (r < a.m_size0 && c < a.m_size1) ? in[r * a.m_stride0 + c * a.m_stride1] : pad;
  }
}

// One thread per element of the matrix.
template <typename T>
__global__ __launch_bounds__(256) void unpack_generic_kernel(PackArgs a) {
  const int64_t total = a.m_size0 * a.m_size1;
  const T* tiled = (const T*)a.out;
  T* mat = (T*)a.in;
  const int tile_rows = a.transpose_inner ? a.t_size3 : a.t_size2;
  const int tile_cols = a.transpose_inner ? a.t_size2 : a.t_size3;
  const int64_t tile_elems = (int64_t)a.t_size2 * a.t_size3;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = idx / a.m_size1, c = idx - r * a.m_size1;
    const int64_t orow = r / tile_rows, ocol = c / tile_cols;
    const int trow = (int)(r - orow * tile_rows), tcol = (int)(c - ocol * tile_cols);
    const int64_t d0 = a.transpose_outer ? ocol : orow, d1 = a.transpose_outer ? orow : ocol;
    const int d2 = a.transpose_inner ? tcol : trow, d3 = a.transpose_inner ? trow : tcol;
    mat[r * a.m_stride0 + c * a.m_stride1] =
        tiled[d0 * a.t_stride0 + d1 * tile_elems + (int64_t)d2 * a.t_size3 + d3];
  }
}

//---------------------------------------------------------------------------
// Streaming kernels. Geometry (all in 16-byte chunks, CE = 16/ES elements):
//   cpr  = chunks per tile row  = tile_cols / CE
//   a "row of chunks" of the matrix has ceil(m_size1 / CE) chunks; chunk j of
//   matrix row r lives in tile column j / cpr, tile row r % tile_rows.
//---------------------------------------------------------------------------

constexpr int kStreamThreads = 256;
constexpr int kStreamUnroll = 4;

struct StreamArgs {
  const char* mat;
  char* tiled;
  int64_t m_size0, m_size1, m_stride0;  // elements
  int64_t outer_rows, outer_cols;       // tile grid in matrix orientation
  int64_t t_stride_row, t_stride_col;   // elements between tiles along matrix rows / cols
  int tile_rows, tile_cols;             // matrix orientation (== stored order)
  int cpr;                              // chunks per tile row
  uint64_t padding;
  int64_t units;                        // work units (see kernels)
};

// pack: a work unit is one wave-sized run of 64 consecutive chunks of the tiled
// buffer inside one outer row of tiles; a wave takes kStreamUnroll consecutive
// runs. Consecutive chunks run along (tile column, tile row, chunk in row), so
// 64 chunks are 1 KiB of contiguous destination.
template <int ES>
__global__ __launch_bounds__(kStreamThreads) void pack_stream_kernel(StreamArgs a) {
  constexpr int CE = 16 / ES;
  typedef typename Chunk<ES>::aligned_t src_vec_t;
  const int lane = threadIdx.x & 63;
  const int64_t wave = ((int64_t)blockIdx.x * kStreamThreads + threadIdx.x) >> 6;
  const int64_t chunks_per_tile = (int64_t)a.tile_rows * a.cpr;
  const int64_t chunks_per_panel = a.outer_cols * chunks_per_tile;
  const int64_t runs_per_panel = ceil_div(chunks_per_panel, 64);
  u32x4 pad_vec;
  {
    uint64_t p = a.padding;
    if (ES == 1) { p &= 0xFF; p |= p << 8; p |= p << 16; p |= p << 32; }
    if (ES == 2) { p &= 0xFFFF; p |= p << 16; p |= p << 32; }
    if (ES == 4) { p &= 0xFFFFFFFFull; p |= p << 32; }
    pad_vec = u32x4{(uint32_t)p, (uint32_t)(p >> 32), (uint32_t)p, (uint32_t)(p >> 32)};
  }
  u32x4 v[kStreamUnroll];
  char* dst[kStreamUnroll];
#pragma unroll
  for (int u = 0; u < kStreamUnroll; ++u) {
    dst[u] = nullptr;
    const int64_t unit = wave * kStreamUnroll + u;
    if (unit >= a.units) continue;
    const int64_t panel = unit / runs_per_panel;
    const int64_t q = (unit - panel * runs_per_panel) * 64 + lane;  // chunk in panel
    if (q >= chunks_per_panel) continue;
    const int64_t tile_col = q / chunks_per_tile;
    const int in_tile = (int)(q - tile_col * chunks_per_tile);
    const int trow = in_tile / a.cpr, h = in_tile - trow * a.cpr;
    const int64_t r = panel * a.tile_rows + trow;
    const int64_t c = tile_col * a.tile_cols + (int64_t)h * CE;
    dst[u] = a.tiled + (panel * a.t_stride_row + tile_col * a.t_stride_col +
                        (int64_t)in_tile * CE) * ES;
    v[u] = pad_vec;
    if (r < a.m_size0 && c < a.m_size1) {
      const char* src = a.mat + (r * a.m_stride0 + c) * ES;
      if (c + CE <= a.m_size1) {
        v[u] = *(const src_vec_t*)src;
      } else {
        // Chunk straddles the right edge: element-wise, never reading past it.
        union { u32x4 vec; uint8_t b[16]; } tmp;
        tmp.vec = pad_vec;
        const int valid = (int)(a.m_size1 - c) * ES;
        for (int i = 0; i < valid; ++i) tmp.b[i] = ((const uint8_t*)src)[i];
        v[u] = tmp.vec;
      }
    }
  }
#pragma unroll
  for (int u = 0; u < kStreamUnroll; ++u)
    if (dst[u]) *(u32x4*)dst[u] = v[u];
}

// unpack: a work unit is 64 consecutive chunks of one matrix row; a wave takes
// kStreamUnroll consecutive ROWS at the same columns (they sit in the same
// tiles, hence the same source cache lines).
template <int ES>
__global__ __launch_bounds__(kStreamThreads) void unpack_stream_kernel(StreamArgs a) {
  constexpr int CE = 16 / ES;
  typedef typename Chunk<ES>::aligned_t dst_vec_t;
  const int lane = threadIdx.x & 63;
  const int64_t wave = ((int64_t)blockIdx.x * kStreamThreads + threadIdx.x) >> 6;
  const int64_t chunks_per_row = ceil_div(a.m_size1, CE);
  const int64_t runs_per_row = ceil_div(chunks_per_row, 64);
  const int64_t row_groups = ceil_div(a.m_size0, kStreamUnroll);
  if (wave >= row_groups * runs_per_row) return;
  const int64_t rg = wave / runs_per_row;
  const int64_t j = (wave - rg * runs_per_row) * 64 + lane;  // chunk in row
  if (j >= chunks_per_row) return;
  const int64_t c = j * CE;
  const int64_t tile_col = j / a.cpr;
  const int h = (int)(j - tile_col * a.cpr);
  u32x4 v[kStreamUnroll];
#pragma unroll
  for (int u = 0; u < kStreamUnroll; ++u) {
    const int64_t r = rg * kStreamUnroll + u;
    if (r >= a.m_size0) continue;
    const int64_t panel = r / a.tile_rows;
    const int trow = (int)(r - panel * a.tile_rows);
    const char* src = a.tiled + (panel * a.t_stride_row + tile_col * a.t_stride_col +
                                 ((int64_t)trow * a.cpr + h) * CE) * ES;
    v[u] = *(const u32x4*)src;
  }
#pragma unroll
  for (int u = 0; u < kStreamUnroll; ++u) {
    const int64_t r = rg * kStreamUnroll + u;
    if (r >= a.m_size0) continue;
    char* dst = (char*)a.mat + (r * a.m_stride0 + c) * ES;
    if (c + CE <= a.m_size1) {
      *(dst_vec_t*)dst = v[u];
    } else {
      union { u32x4 vec; uint8_t b[16]; } tmp;
      tmp.vec = v[u];
      const int valid = (int)(a.m_size1 - c) * ES;
      for (int i = 0; i < valid; ++i) ((uint8_t*)dst)[i] = tmp.b[i];
    }
  }
}

bool stream_eligible(int es, int64_t m_stride1, int transpose_inner, int tile_cols,
                     const void* tiled, int64_t t_stride0, int64_t tile_elems) {
  const int ce = 16 / es;
  return m_stride1 == 1 && !transpose_inner && tile_cols > 0 && tile_cols % ce == 0 &&
         ((uintptr_t)tiled % 16) == 0 && (t_stride0 * es) % 16 == 0 &&
         (tile_elems * es) % 16 == 0;
}

template <int ES>
int launch_pack_stream(const StreamArgs& a, hipStream_t s) {
  const int64_t waves = ceil_div(a.units, kStreamUnroll);
  const int64_t blocks = ceil_div(waves, kStreamThreads / 64);
  if (blocks > 0x7FFFFFFF) return IREE_AMD_UK_STATUS_NOT_FOUND;
  hipLaunchKernelGGL(pack_stream_kernel<ES>, dim3((unsigned)blocks), dim3(kStreamThreads), 0, s, a);
  return check_hip(hipGetLastError(), "pack_stream launch");
}

template <int ES>
int launch_unpack_stream(const StreamArgs& a, hipStream_t s) {
  constexpr int CE = 16 / ES;
  const int64_t waves = ceil_div(a.m_size0, kStreamUnroll) * ceil_div(ceil_div(a.m_size1, CE), 64);
  const int64_t blocks = ceil_div(waves, kStreamThreads / 64);
  if (blocks > 0x7FFFFFFF) return IREE_AMD_UK_STATUS_NOT_FOUND;
  hipLaunchKernelGGL(unpack_stream_kernel<ES>, dim3((unsigned)blocks), dim3(kStreamThreads), 0, s, a);
  return check_hip(hipGetLastError(), "unpack_stream launch");
}

template <typename T, typename K>
int launch_generic(K kernel, const PackArgs& a, int64_t total, hipStream_t s, const char* what) {
  int64_t blocks = ceil_div(total, 256);
  const int64_t max_blocks = (int64_t)device_cu_count() * 64;
  if (blocks > max_blocks) blocks = max_blocks;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(256), 0, s, a);
  return check_hip(hipGetLastError(), what);
}

}  // namespace

int launch_pack(const iree_amd_uk_pack_params_t& p, hipStream_t s) {
  const int es = pack_elem_bytes(p.flags);
  const int ti = (p.flags & IREE_AMD_UK_FLAG_PACK_TRANSPOSE_INNER) != 0;
  const int to = (p.flags & IREE_AMD_UK_FLAG_PACK_TRANSPOSE_OUTER) != 0;
  const char* in = (const char*)p.in_buffer + p.in_offset * es;
  char* out = (char*)p.out_buffer + p.out_offset * es;
  const int64_t tile_elems = p.out_size2 * p.out_size3;
  if (p.out_size2 > 0x7FFFFFFF || p.out_size3 > 0x7FFFFFFF || tile_elems > 0x7FFFFFFF)
    return fail(IREE_AMD_UK_STATUS_OUT_OF_RANGE, "pack: tile larger than 2^31 elements");

  if (stream_eligible(es, p.in_stride1, ti, (int)p.out_size3, out, p.out_stride0, tile_elems)) {
    StreamArgs a;
    a.mat = in; a.tiled = out;
    a.m_size0 = p.in_size0; a.m_size1 = p.in_size1; a.m_stride0 = p.in_stride0;
    a.outer_rows = to ? p.out_size1 : p.out_size0;
    a.outer_cols = to ? p.out_size0 : p.out_size1;
    a.t_stride_row = to ? tile_elems : p.out_stride0;
    a.t_stride_col = to ? p.out_stride0 : tile_elems;
    a.tile_rows = (int)p.out_size2; a.tile_cols = (int)p.out_size3;
    a.cpr = a.tile_cols / (16 / es);
    a.padding = p.padding_value;
    const int64_t chunks_per_panel = a.outer_cols * (int64_t)a.tile_rows * a.cpr;
    a.units = a.outer_rows * ceil_div(chunks_per_panel, 64);
    // With swapped outer dimensions consecutive tile columns are t_stride0
    // apart; the 1 KiB runs then only stay contiguous inside one tile, which
    // is still a whole number of chunks.
    int st = es == 1 ? launch_pack_stream<1>(a, s)
           : es == 2 ? launch_pack_stream<2>(a, s)
                     : launch_pack_stream<4>(a, s);
    if (st != IREE_AMD_UK_STATUS_NOT_FOUND) return st;
  }

  PackArgs a;
  a.in = in; a.out = out;
  a.m_size0 = p.in_size0; a.m_size1 = p.in_size1;
  a.m_stride0 = p.in_stride0; a.m_stride1 = p.in_stride1;
  a.t_size0 = p.out_size0; a.t_size1 = p.out_size1; a.t_stride0 = p.out_stride0;
  a.t_size2 = (int)p.out_size2; a.t_size3 = (int)p.out_size3;
  a.transpose_inner = ti; a.transpose_outer = to; a.padding = p.padding_value;
  const int64_t total = p.out_size0 * p.out_size1 * tile_elems;
  switch (es) {
    case 1: return launch_generic<uint8_t>(pack_generic_kernel<uint8_t>, a, total, s, "pack_generic launch");
    case 2: return launch_generic<uint16_t>(pack_generic_kernel<uint16_t>, a, total, s, "pack_generic launch");
    default: return launch_generic<uint32_t>(pack_generic_kernel<uint32_t>, a, total, s, "pack_generic launch");
  }
}

int launch_unpack(const iree_amd_uk_unpack_params_t& p, hipStream_t s) {
  const int es = unpack_elem_bytes(p.flags);
  const int ti = (p.flags & IREE_AMD_UK_FLAG_UNPACK_TRANSPOSE_INNER) != 0;
  const int to = (p.flags & IREE_AMD_UK_FLAG_UNPACK_TRANSPOSE_OUTER) != 0;
  const char* tiled = (const char*)p.in_buffer + p.in_offset * es;
  char* mat = (char*)p.out_buffer + p.out_offset * es;
  const int64_t tile_elems = p.in_size2 * p.in_size3;
  if (p.in_size2 > 0x7FFFFFFF || p.in_size3 > 0x7FFFFFFF || tile_elems > 0x7FFFFFFF)
    return fail(IREE_AMD_UK_STATUS_OUT_OF_RANGE, "unpack: tile larger than 2^31 elements");
  if (tile_elems == 0) return 0;  // validated: then out sizes are 0 too

  if (stream_eligible(es, p.out_stride1, ti, (int)p.in_size3, tiled, p.in_stride0, tile_elems)) {
    StreamArgs a;
    a.mat = mat; a.tiled = (char*)tiled;
    a.m_size0 = p.out_size0; a.m_size1 = p.out_size1; a.m_stride0 = p.out_stride0;
    a.outer_rows = to ? p.in_size1 : p.in_size0;
    a.outer_cols = to ? p.in_size0 : p.in_size1;
    a.t_stride_row = to ? tile_elems : p.in_stride0;
    a.t_stride_col = to ? p.in_stride0 : tile_elems;
    a.tile_rows = (int)p.in_size2; a.tile_cols = (int)p.in_size3;
    a.cpr = a.tile_cols / (16 / es);
    a.padding = 0; a.units = 0;
    int st = es == 2 ? launch_unpack_stream<2>(a, s) : launch_unpack_stream<4>(a, s);
    if (st != IREE_AMD_UK_STATUS_NOT_FOUND) return st;
  }

  PackArgs a;
  a.in = mat; a.out = (char*)tiled;
  a.m_size0 = p.out_size0; a.m_size1 = p.out_size1;
  a.m_stride0 = p.out_stride0; a.m_stride1 = p.out_stride1;
  a.t_size0 = p.in_size0; a.t_size1 = p.in_size1; a.t_stride0 = p.in_stride0;
  a.t_size2 = (int)p.in_size2; a.t_size3 = (int)p.in_size3;
  a.transpose_inner = ti; a.transpose_outer = to; a.padding = 0;
  const int64_t total = p.out_size0 * p.out_size1;
  switch (es) {
    case 2: return launch_generic<uint16_t>(unpack_generic_kernel<uint16_t>, a, total, s, "unpack_generic launch");
    default: return launch_generic<uint32_t>(unpack_generic_kernel<uint32_t>, a, total, s, "unpack_generic launch");
  }
}

}  // namespace uk
