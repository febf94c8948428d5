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
#include "uk_pack_stream_kernel.h"
#include "uk_pack_transpose_kernel.h"

namespace uk {
namespace {

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
// All per-lane index arithmetic is 32-bit; divisions by run-time constants go
// through a precomputed multiply-shift. The grid's y dimension walks the outer
// rows of tiles (pack) or groups of matrix rows (unpack).
//---------------------------------------------------------------------------


struct StreamArgs {
  const char* mat;
  char* tiled;
  int64_t m_size0, m_size1, m_stride0;  // elements
  int64_t outer_rows, outer_cols;       // tile grid in matrix orientation
  int64_t t_stride_row, t_stride_col;   // elements between tiles along matrix rows / cols
  int tile_rows, tile_cols;             // matrix orientation (== stored order)
  int cpr;                              // chunks per tile row
  uint32_t chunks_per_row;              // ceil(m_size1 / CE)
  uint32_t padded_chunks_per_row;       // outer_cols * cpr
  int64_t padded_rows;                  // outer_rows * tile_rows
  int64_t t_stride_row_bytes, t_stride_col_bytes;
  int log2_tile_rows, log2_cpr;         // valid when both are powers of two
  int pow2;
  FastDiv by_cpr, by_tile_rows;
  uint64_t padding;
};


// Position of matrix element (row r, chunk column j) in the tiled buffer, in
// bytes from the buffer start. kPow2: tile_rows and cpr are powers of two (every
// gfx950 tile shape is) and the divisions become shifts.
template <bool kPow2>
__device__ __forceinline__ int64_t tiled_chunk_offset(const StreamArgs& a, int64_t r, uint32_t j) {
  int64_t panel;
  uint32_t trow, tile_col, h;
  if (kPow2) {
    panel = r >> a.log2_tile_rows;
    trow = (uint32_t)r & (a.tile_rows - 1);
    tile_col = j >> a.log2_cpr;
    h = j & (a.cpr - 1);
  } else {
    if (r < 0x7FFFFFFF) {
      panel = a.by_tile_rows.div((uint32_t)r);
      trow = (uint32_t)r - (uint32_t)panel * a.tile_rows;
    } else {
      panel = r / a.tile_rows;
      trow = (uint32_t)(r - panel * a.tile_rows);
    }
    tile_col = a.by_cpr.div(j);
    h = j - tile_col * a.cpr;
  }
  return panel * a.t_stride_row_bytes + (int64_t)tile_col * a.t_stride_col_bytes +
         (int64_t)(trow * a.cpr + h) * 16;
}

template <int ES, bool kPow2>
__global__ __launch_bounds__(kStreamThreads) void pack_stream_kernel(StreamArgs a) {
  constexpr int CE = 16 / ES;
  typedef typename Chunk<ES>::aligned_t src_vec_t;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t j0 = (blockIdx.x * 4 + wave) * kBlockChunks;   // first chunk column of the wave
  if (j0 >= a.padded_chunks_per_row) return;
  const uint32_t j = j0 + (lane & 7);
  const int64_t c = (int64_t)j * CE;
  const int64_t row_groups = ceil_div(a.padded_rows, kBlockRows * kStreamUnroll);
  // Wave-uniform: every chunk of the strip lies wholly inside the matrix.
  const bool cols_inside = (int64_t)(j0 + kBlockChunks) * CE <= a.m_size1;
  for (int64_t rg = blockIdx.y; rg < row_groups; rg += gridDim.y) {
    const int64_t r0 = rg * kStreamUnroll * kBlockRows;
    if (cols_inside && r0 + kStreamUnroll * kBlockRows <= a.m_size0) {
      // Interior: straight-line code, all loads in flight before the stores.
      u32x4 v[kStreamUnroll];
#pragma unroll
      for (int u = 0; u < kStreamUnroll; ++u) {
        const int64_t r = r0 + u * kBlockRows + (lane >> 3);
        v[u] = *(const src_vec_t*)(a.mat + (r * a.m_stride0 + c) * ES);
      }
#pragma unroll
      for (int u = 0; u < kStreamUnroll; ++u) {
        const int64_t r = r0 + u * kBlockRows + (lane >> 3);
        *(u32x4*)(a.tiled + tiled_chunk_offset<kPow2>(a, r, j)) = v[u];
      }
      continue;
    }
    // Edge: per-lane predicates, padding, and a byte-wise tail for the chunk
    // that straddles the right edge (never reading past it).
    u32x4 pad_vec;
    {
      uint64_t p = a.padding;
      if (ES == 1) { p &= 0xFF; p |= p << 8; p |= p << 16; p |= p << 32; }
      if (ES == 2) { p &= 0xFFFF; p |= p << 16; p |= p << 32; }
      if (ES == 4) { p &= 0xFFFFFFFFull; p |= p << 32; }
      pad_vec = u32x4{(uint32_t)p, (uint32_t)(p >> 32), (uint32_t)p, (uint32_t)(p >> 32)};
    }
    if (j >= a.padded_chunks_per_row) continue;
#pragma unroll 1
    for (int u = 0; u < kStreamUnroll; ++u) {
      const int64_t r = r0 + u * kBlockRows + (lane >> 3);
      if (r >= a.padded_rows) continue;
      u32x4 v = pad_vec;
      if (r < a.m_size0 && c < a.m_size1) {
        const char* src = a.mat + (r * a.m_stride0 + c) * ES;
        if (c + CE <= a.m_size1) {
          v = *(const src_vec_t*)src;
        } else {
          union { u32x4 vec; uint8_t b[16]; } tmp;
          tmp.vec = pad_vec;
          const int valid = (int)(a.m_size1 - c) * ES;
          for (int i = 0; i < valid; ++i) tmp.b[i] = ((const uint8_t*)src)[i];
          v = tmp.vec;
        }
      }
      *(u32x4*)(a.tiled + tiled_chunk_offset<kPow2>(a, r, j)) = v;
    }
  }
}

template <int ES, bool kPow2>
__global__ __launch_bounds__(kStreamThreads) void unpack_stream_kernel(StreamArgs a) {
  constexpr int CE = 16 / ES;
  typedef typename Chunk<ES>::aligned_t dst_vec_t;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t j0 = (blockIdx.x * 4 + wave) * kBlockChunks;
  if (j0 >= a.chunks_per_row) return;
  const uint32_t j = j0 + (lane & 7);
  const int64_t c = (int64_t)j * CE;
  const int64_t row_groups = ceil_div(a.m_size0, kBlockRows * kStreamUnroll);
  const bool cols_inside = (int64_t)(j0 + kBlockChunks) * CE <= a.m_size1;
  for (int64_t rg = blockIdx.y; rg < row_groups; rg += gridDim.y) {
    const int64_t r0 = rg * kStreamUnroll * kBlockRows;
    if (cols_inside && r0 + kStreamUnroll * kBlockRows <= a.m_size0) {
      u32x4 v[kStreamUnroll];
#pragma unroll
      for (int u = 0; u < kStreamUnroll; ++u) {
        const int64_t r = r0 + u * kBlockRows + (lane >> 3);
        v[u] = *(const u32x4*)(a.tiled + tiled_chunk_offset<kPow2>(a, r, j));
      }
#pragma unroll
      for (int u = 0; u < kStreamUnroll; ++u) {
        const int64_t r = r0 + u * kBlockRows + (lane >> 3);
        *(dst_vec_t*)((char*)a.mat + (r * a.m_stride0 + c) * ES) = v[u];
      }
      continue;
    }
    if (j >= a.chunks_per_row) continue;
#pragma unroll 1
    for (int u = 0; u < kStreamUnroll; ++u) {
      const int64_t r = r0 + u * kBlockRows + (lane >> 3);
      if (r >= a.m_size0) continue;
      const u32x4 v = *(const u32x4*)(a.tiled + tiled_chunk_offset<kPow2>(a, r, j));
      char* dst = (char*)a.mat + (r * a.m_stride0 + c) * ES;
      if (c + CE <= a.m_size1) {
        *(dst_vec_t*)dst = v;
      } else {
        union { u32x4 vec; uint8_t b[16]; } tmp;
        tmp.vec = v;
        const int valid = (int)(a.m_size1 - c) * ES;
        for (int i = 0; i < valid; ++i) ((uint8_t*)dst)[i] = tmp.b[i];
      }
    }
  }
}

template <int ES, bool kPack, int kRows = kPow2Rows>
__global__ __launch_bounds__(kPow2Waves * 64) void stream_pow2_kernel(Pow2Args a) {
  stream_pow2_body<ES, kPack, true, kPack, kRows>(a);
}

// The 32-bit per-lane offsets of stream_pow2_kernel must not overflow.
bool pow2_eligible(const StreamArgs& a, int es) {
  if (!a.pow2) return false;
  const int64_t rows = 8 * kPow2Unroll;      // (the taller of the two block shapes)
  const int64_t pitch = a.m_stride0 * es;
  if (pitch * rows + 256 >= (1ll << 31)) return false;
  const int64_t panels = rows / a.tile_rows + 2, cols = (64 / kPow2Rows) / a.cpr + 2;
  if (a.t_stride_row_bytes * panels + a.t_stride_col_bytes * cols + (1ll << 20) >= (1ll << 31)) return false;
  if ((int64_t)a.tile_rows * a.cpr * 16 >= (1ll << 20)) return false;
  return true;
}

template <int ES, bool kPack>
int launch_stream_pow2(const StreamArgs& a, hipStream_t s) {
  Pow2Args p;
  p.mat = a.mat; p.tiled = a.tiled;
  p.m_size0 = a.m_size0; p.m_size1 = a.m_size1; p.m_pitch_bytes = a.m_stride0 * ES;
  p.t_stride_row_bytes = a.t_stride_row_bytes; p.t_stride_col_bytes = a.t_stride_col_bytes;
  p.padded_rows = a.padded_rows;
  p.chunks_per_row = a.chunks_per_row; p.padded_chunks_per_row = a.padded_chunks_per_row;
  p.log2_tile_rows = a.log2_tile_rows; p.log2_cpr = a.log2_cpr;
  p.padding = a.padding;
  const int64_t cols = kPack ? a.padded_chunks_per_row : a.chunks_per_row;
  const int64_t rows = kPack ? a.padded_rows : a.m_size0;
  // Tiles whose rows are a single chunk (f16 32x8, i8 32x16, f32 32x4: the
  // operand tiles of mmt4d): 8 rows x 8 chunks per wave, so that the wave's
  // piece of a tile is a whole 128-byte line (4 rows x 16 chunks leave half of
  // each line to the wave below, and both sides are accessed non-temporally).
  // Measured (TB/s, 4 rows x 16 chunks -> 8 x 8): pack i8 8192^2 into 32x16
  // 4.75 -> 5.62, f16 8192 x 4096 into 32x8 4.75 -> 5.62, f32 4096^2 into 32x4
  // 4.50 -> 5.55; unpack f16 from 32x8 5.65 -> 6.09 (8191 x 5001: 5.02 -> 5.20).
  const bool tall = a.cpr == 1 && a.tile_rows >= 8;
  const int block_rows = tall ? 8 : kPow2Rows;
  const int64_t bx = ceil_div(cols, kPow2WavesX * (64 / block_rows));
  const int64_t by = ceil_div(rows, block_rows * kPow2Unroll * (kPow2Waves / kPow2WavesX));
  if (bx < 1 || by < 1 || bx * by > 0x7FFFFFFF) return IREE_AMD_UK_STATUS_NOT_FOUND;
  p.blocks_x = (uint32_t)bx; p.blocks_y = (uint32_t)by;
  if (tall)
    hipLaunchKernelGGL((stream_pow2_kernel<ES, kPack, 8>), dim3((unsigned)(bx * by)), dim3(kPow2Waves * 64), 0, s, p);
  else
    hipLaunchKernelGGL((stream_pow2_kernel<ES, kPack>), dim3((unsigned)(bx * by)), dim3(kPow2Waves * 64), 0, s, p);
  return check_hip(hipGetLastError(), "stream_pow2 launch");
}

template <int ES>
__global__ __launch_bounds__(256) void pack_transpose_kernel(TransArgs a) { pack_transpose_body<ES>(a); }
template <int ES>
__global__ __launch_bounds__(256) void unpack_transpose_kernel(TransArgs a) { unpack_transpose_body<ES>(a); }
template <int ES>
__global__ __launch_bounds__(256) void pack_transpose_wide_kernel(TransArgs a) { pack_transpose_wide_body<ES>(a); }
template <int ES, int kLdsUnroll>
__global__ __launch_bounds__(256) void pack_transpose_lds_kernel(TransArgs a) {
  pack_transpose_lds_body<ES, kLdsUnroll>(a);
}

template <int ES, int kLX, bool kNt = false>
__global__ __launch_bounds__(64) void unpack_transpose_block_kernel(TransArgs a) {
  unpack_transpose_block_body<ES, kLX, kNt>(a);
}

template <int ES>
int launch_unpack_transpose(TransArgs a, hipStream_t s) {
  const int64_t cols = a.m_size1 < a.padded_cols ? a.m_size1 : a.padded_cols;
  // Tiles of whole CE columns and enough columns for a wave's 16 blocks: the
  // kernel that moves a CE x CE block per lane, one wave per workgroup.
  constexpr int CE = 16 / ES;
  if (a.tile_cols % CE == 0 && cols >= 16 * CE) {
    // Tiles of 8 row groups and more (stored columns of at least 128 bytes): a
    // wave takes 8 blocks across and 8 row groups, so that it consumes whole
    // lines of the stored columns by itself (16 across and 4 row groups leave
    // the other half of every line to another wave, and a line that two waves
    // load non-temporally comes from memory twice: 1.15 x the traffic). f32
    // 4096 x 4096 from 32x32 tiles: 27.1 -> 24.3 us.
    const bool tall = a.groups_per_tile % 8 == 0;
    const int lx = tall ? 8 : 16, gy = 64 / lx;
    const int64_t bx = ceil_div(cols, (int64_t)lx * CE);
    const int64_t by = ceil_div(a.row_groups, (int64_t)gy);
    if (bx >= 1 && by >= 1 && bx * by <= 0x7FFFFFFF) {
      a.blocks_x = (uint32_t)bx; a.blocks_y = (uint32_t)by;
      if (tall) hipLaunchKernelGGL((unpack_transpose_block_kernel<ES, 8>), dim3((unsigned)(bx * by)), dim3(64), 0, s, a);
      else hipLaunchKernelGGL((unpack_transpose_block_kernel<ES, 16>), dim3((unsigned)(bx * by)), dim3(64), 0, s, a);
      return check_hip(hipGetLastError(), "unpack_transpose launch");
    }
  }
  const int64_t bx = ceil_div(cols, (int64_t)64);
  const int64_t by = ceil_div(a.row_groups, (int64_t)(4 * kTransUnroll));
  if (bx < 1 || by < 1 || bx * by > 0x7FFFFFFF) return IREE_AMD_UK_STATUS_NOT_FOUND;
  a.blocks_x = (uint32_t)bx; a.blocks_y = (uint32_t)by;
  hipLaunchKernelGGL((unpack_transpose_kernel<ES>), dim3((unsigned)(bx * by)), dim3(256), 0, s, a);
  return check_hip(hipGetLastError(), "unpack_transpose launch");
}

template <int ES>
int launch_pack_transpose(TransArgs a, hipStream_t s) {
  // 1- and 2-byte elements: dword loads where every row starts on a 4-byte
  // boundary and tiles are whole dwords of columns
  constexpr int W = ES < 4 ? 4 / ES : 1;
  const bool wide = W > 1 && a.tile_cols % W == 0 && (uintptr_t)a.mat % 4 == 0 && a.m_pitch_bytes % 4 == 0;
  // 2-byte elements, 512 columns and more in tiles of whole 8 columns: 16-byte
  // loads and an exchange through LDS, 4 row groups per wave where that still
  // gives every compute unit a workgroup, else 1 (small matrices keep the
  // finer-grained kernels below)
  if constexpr (ES == 2) {
    if (wide && a.tile_cols % 8 == 0 && a.padded_cols >= 512) {
      const int64_t lx = ceil_div(a.padded_cols, (int64_t)512);
      const int64_t ly4 = ceil_div(a.row_groups, (int64_t)16), ly1 = ceil_div(a.row_groups, (int64_t)4);
      const int cus = device_cu_count();
      if (lx * ly4 >= cus && lx * ly4 <= 0x7FFFFFFF) {
        a.blocks_x = (uint32_t)lx; a.blocks_y = (uint32_t)ly4;
        hipLaunchKernelGGL((pack_transpose_lds_kernel<ES, 4>), dim3((unsigned)(lx * ly4)), dim3(256), 0, s, a);
        return check_hip(hipGetLastError(), "pack_transpose launch");
      }
      if (lx * ly1 >= cus && lx * ly1 <= 0x7FFFFFFF) {
        a.blocks_x = (uint32_t)lx; a.blocks_y = (uint32_t)ly1;
        hipLaunchKernelGGL((pack_transpose_lds_kernel<ES, 1>), dim3((unsigned)(lx * ly1)), dim3(256), 0, s, a);
        return check_hip(hipGetLastError(), "pack_transpose launch");
      }
    }
  }
  const int64_t bx = ceil_div(a.padded_cols, (int64_t)64 * (wide ? W : 1));
  const int64_t by = ceil_div(a.row_groups, (int64_t)(4 * kTransUnroll));
  if (bx < 1 || by < 1 || bx * by > 0x7FFFFFFF) return IREE_AMD_UK_STATUS_NOT_FOUND;
  a.blocks_x = (uint32_t)bx; a.blocks_y = (uint32_t)by;
  if constexpr (W > 1) {
    if (wide) {
      hipLaunchKernelGGL((pack_transpose_wide_kernel<ES>), dim3((unsigned)(bx * by)), dim3(256), 0, s, a);
      return check_hip(hipGetLastError(), "pack_transpose launch");
    }
  }
  hipLaunchKernelGGL((pack_transpose_kernel<ES>), dim3((unsigned)(bx * by)), dim3(256), 0, s, a);
  return check_hip(hipGetLastError(), "pack_transpose launch");
}

bool stream_eligible(int es, int64_t m_stride1, int transpose_inner, int64_t tile_rows,
                     int64_t tile_cols, int64_t outer_cols, int64_t m_size1, const void* tiled,
                     int64_t t_stride0, int64_t tile_elems) {
  const int ce = 16 / es;
  if (!(m_stride1 == 1 && !transpose_inner && tile_cols > 0 && tile_cols % ce == 0 &&
        ((uintptr_t)tiled % 16) == 0 && (t_stride0 * es) % 16 == 0 && (tile_elems * es) % 16 == 0))
    return false;
  // 32-bit per-lane column arithmetic: chunks per row must stay below 2^31.
  return tile_rows < (1ll << 31) && outer_cols * (tile_cols / ce) < (1ll << 31) &&
         m_size1 / ce + 1 < (1ll << 31);
}

void fill_stream_geometry(StreamArgs* a, int es) {
  const int ce = 16 / es;
  a->cpr = a->tile_cols / ce;
  a->chunks_per_row = (uint32_t)((a->m_size1 + ce - 1) / ce);
  a->padded_chunks_per_row = (uint32_t)(a->outer_cols * a->cpr);
  a->padded_rows = a->outer_rows * a->tile_rows;
  a->t_stride_row_bytes = a->t_stride_row * es;
  a->t_stride_col_bytes = a->t_stride_col * es;
  a->by_cpr = make_fastdiv((uint32_t)a->cpr);
  a->by_tile_rows = make_fastdiv((uint32_t)a->tile_rows);
  auto is_pow2 = [](int v) { return v > 0 && (v & (v - 1)) == 0; };
  a->pow2 = is_pow2(a->tile_rows) && is_pow2(a->cpr);
  a->log2_tile_rows = a->log2_cpr = 0;
  while ((1 << a->log2_tile_rows) < a->tile_rows) ++a->log2_tile_rows;
  while ((1 << a->log2_cpr) < a->cpr) ++a->log2_cpr;
}

template <int ES>
int launch_pack_stream(const StreamArgs& a, hipStream_t s) {
  if (pow2_eligible(a, ES)) return launch_stream_pow2<ES, true>(a, s);
  const int64_t bx = ceil_div(a.padded_chunks_per_row, 4 * kBlockChunks);
  const int64_t row_groups = ceil_div(a.padded_rows, kBlockRows * kStreamUnroll);
  const int64_t by = row_groups < 65535 ? row_groups : 65535;
  if (bx > 0x7FFFFFFF) return IREE_AMD_UK_STATUS_NOT_FOUND;
  if (a.pow2)
    hipLaunchKernelGGL((pack_stream_kernel<ES, true>), dim3((unsigned)bx, (unsigned)by), dim3(kStreamThreads), 0, s, a);
  else
    hipLaunchKernelGGL((pack_stream_kernel<ES, false>), dim3((unsigned)bx, (unsigned)by), dim3(kStreamThreads), 0, s, a);
  return check_hip(hipGetLastError(), "pack_stream launch");
}

template <int ES>
__global__ __launch_bounds__(64) void unpack_aligned_kernel(Pow2Args a) { unpack_aligned_body<ES>(a); }

// Rows of at least 1 KiB in power-of-two tiles: the kernel whose stores are
// aligned cache lines (one wave per workgroup: 4 rows x one 256-byte window).
template <int ES>
int launch_unpack_aligned(const StreamArgs& a, hipStream_t s) {
  const int64_t row_bytes = a.m_size1 * ES;
  // (32-bit offsets per lane: the same limits as the other power-of-two kernel)
  // (tiles whose rows are a single chunk: 4 rows of one tile are half a line,
  // the other kernel's 8-row blocks read whole ones: 6.09 against 5.41 TB/s
  // for f16 8192 x 4096 from 32x8 tiles)
  if (a.cpr == 1) return IREE_AMD_UK_STATUS_NOT_FOUND;
  // Tile rows of 64 bytes and more: the other kernel's row pieces are then long
  // runs on the tiled side as well (4 rows x 256 bytes of a 32x32 f32 tile are
  // 512 contiguous bytes), and it measures faster than this one, whose windows
  // cut tile rows at arbitrary chunks: f32 4096^2 from 32x32 tiles 5.94 against
  // 5.60 TB/s (4095 x 4099: 6.03 against 5.44), f16 8192 x 4096 from 32x32
  // 6.10 against 5.79. With 32-byte tile rows (f16 32x16) this kernel wins:
  // 6.08 against 5.57 (8191 x 5001: 5.77 against 5.39).
  if (a.cpr >= 4) return IREE_AMD_UK_STATUS_NOT_FOUND;
  if (!pow2_eligible(a, ES) || row_bytes < 1024 || row_bytes + 512 >= (1ll << 31) || a.m_size0 < 1 ||
      a.m_stride0 * ES * 16 + row_bytes + 512 >= (1ll << 31))
    return IREE_AMD_UK_STATUS_NOT_FOUND;
  Pow2Args p;
  p.mat = a.mat; p.tiled = a.tiled;
  p.m_size0 = a.m_size0; p.m_size1 = a.m_size1; p.m_pitch_bytes = a.m_stride0 * ES;
  p.t_stride_row_bytes = a.t_stride_row_bytes; p.t_stride_col_bytes = a.t_stride_col_bytes;
  p.padded_rows = a.padded_rows;
  p.chunks_per_row = a.chunks_per_row; p.padded_chunks_per_row = a.padded_chunks_per_row;
  p.log2_tile_rows = a.log2_tile_rows; p.log2_cpr = a.log2_cpr;
  p.padding = a.padding;
  // windows a row can touch: it starts up to 127 bytes into its first line
  const int64_t bx = (row_bytes + 127 + 255) / 256;
  const int64_t by = ceil_div(a.m_size0, (int64_t)4);
  if (bx * by > 0x7FFFFFFF) return IREE_AMD_UK_STATUS_NOT_FOUND;
  p.blocks_x = (uint32_t)bx; p.blocks_y = (uint32_t)by;
  hipLaunchKernelGGL((unpack_aligned_kernel<ES>), dim3((unsigned)(bx * by)), dim3(64), 0, s, p);
  return check_hip(hipGetLastError(), "unpack_aligned launch");
}

template <int ES>
int launch_unpack_stream(const StreamArgs& a, hipStream_t s) {
  {
    const int st = launch_unpack_aligned<ES>(a, s);
    if (st != IREE_AMD_UK_STATUS_NOT_FOUND) return st;
  }
  if (pow2_eligible(a, ES)) return launch_stream_pow2<ES, false>(a, s);
  const int64_t bx = ceil_div(a.chunks_per_row, 4 * kBlockChunks);
  const int64_t row_groups = ceil_div(a.m_size0, kBlockRows * kStreamUnroll);
  const int64_t by = row_groups < 65535 ? row_groups : 65535;
  if (bx > 0x7FFFFFFF) return IREE_AMD_UK_STATUS_NOT_FOUND;
  if (a.pow2)
    hipLaunchKernelGGL((unpack_stream_kernel<ES, true>), dim3((unsigned)bx, (unsigned)by), dim3(kStreamThreads), 0, s, a);
  else
    hipLaunchKernelGGL((unpack_stream_kernel<ES, false>), dim3((unsigned)bx, (unsigned)by), dim3(kStreamThreads), 0, s, a);
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

  if (stream_eligible(es, p.in_stride1, ti, p.out_size2, p.out_size3, to ? p.out_size0 : p.out_size1,
                      p.in_size1, out, p.out_stride0, tile_elems)) {
    StreamArgs a;
    a.mat = in; a.tiled = out;
    a.m_size0 = p.in_size0; a.m_size1 = p.in_size1; a.m_stride0 = p.in_stride0;
    a.outer_rows = to ? p.out_size1 : p.out_size0;
    a.outer_cols = to ? p.out_size0 : p.out_size1;
    a.t_stride_row = to ? tile_elems : p.out_stride0;
    a.t_stride_col = to ? p.out_stride0 : tile_elems;
    a.tile_rows = (int)p.out_size2; a.tile_cols = (int)p.out_size3;
    a.padding = p.padding_value;
    fill_stream_geometry(&a, es);
    // With swapped outer dimensions consecutive tile columns are t_stride0
    // apart; the 1 KiB runs then only stay contiguous inside one tile, which
    // is still a whole number of chunks.
    int st = es == 1 ? launch_pack_stream<1>(a, s)
           : es == 2 ? launch_pack_stream<2>(a, s)
                     : launch_pack_stream<4>(a, s);
    if (st != IREE_AMD_UK_STATUS_NOT_FOUND) return st;
  }

  // Transposed inner tiles whose stored rows are whole 16-byte chunks.
  const int ce = 16 / es;
  if (ti && p.in_stride1 == 1 && p.out_size3 > 0 && p.out_size3 % ce == 0 && p.out_size2 > 0 &&
      ((uintptr_t)out % 16) == 0 && (p.out_stride0 * es) % 16 == 0 && (tile_elems * es) % 16 == 0 &&
      p.in_size1 < (1ll << 31) && (to ? p.out_size0 : p.out_size1) * p.out_size2 < (1ll << 31)) {
    TransArgs a;
    a.mat = in; a.tiled = out;
    a.m_size0 = p.in_size0; a.m_size1 = p.in_size1; a.m_pitch_bytes = p.in_stride0 * es;
    a.tile_rows = (int)p.out_size3; a.tile_cols = (int)p.out_size2;
    a.groups_per_tile = a.tile_rows / ce;
    const int64_t outer_rows = to ? p.out_size1 : p.out_size0;
    const int64_t outer_cols = to ? p.out_size0 : p.out_size1;
    a.row_groups = outer_rows * a.groups_per_tile;
    a.padded_cols = outer_cols * a.tile_cols;
    a.t_stride_orow_bytes = (to ? tile_elems : p.out_stride0) * es;
    a.t_stride_ocol_bytes = (to ? p.out_stride0 : tile_elems) * es;
    a.by_tile_cols = make_fastdiv((uint32_t)a.tile_cols);
    a.by_groups = make_fastdiv((uint32_t)a.groups_per_tile);
    a.padding = p.padding_value;
    a.blocks_x = a.blocks_y = 0;
    int st = es == 1 ? launch_pack_transpose<1>(a, s)
           : es == 2 ? launch_pack_transpose<2>(a, s)
                     : launch_pack_transpose<4>(a, s);
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

  if (stream_eligible(es, p.out_stride1, ti, p.in_size2, p.in_size3, to ? p.in_size0 : p.in_size1,
                      p.out_size1, tiled, p.in_stride0, tile_elems)) {
    StreamArgs a;
    a.mat = mat; a.tiled = (char*)tiled;
    a.m_size0 = p.out_size0; a.m_size1 = p.out_size1; a.m_stride0 = p.out_stride0;
    a.outer_rows = to ? p.in_size1 : p.in_size0;
    a.outer_cols = to ? p.in_size0 : p.in_size1;
    a.t_stride_row = to ? tile_elems : p.in_stride0;
    a.t_stride_col = to ? p.in_stride0 : tile_elems;
    a.tile_rows = (int)p.in_size2; a.tile_cols = (int)p.in_size3;
    a.padding = 0;
    fill_stream_geometry(&a, es);
    int st = es == 2 ? launch_unpack_stream<2>(a, s) : launch_unpack_stream<4>(a, s);
    if (st != IREE_AMD_UK_STATUS_NOT_FOUND) return st;
  }

  // Transposed inner tiles whose stored rows are whole 16-byte chunks.
  const int ce = 16 / es;
  if (ti && p.out_stride1 == 1 && p.in_size3 > 0 && p.in_size3 % ce == 0 && p.in_size2 > 0 &&
      ((uintptr_t)tiled % 16) == 0 && (p.in_stride0 * es) % 16 == 0 && (tile_elems * es) % 16 == 0 &&
      p.out_size1 < (1ll << 31) && (to ? p.in_size0 : p.in_size1) * p.in_size2 < (1ll << 31)) {
    TransArgs a;
    a.mat = mat; a.tiled = (char*)tiled;
    a.m_size0 = p.out_size0; a.m_size1 = p.out_size1; a.m_pitch_bytes = p.out_stride0 * es;
    a.tile_rows = (int)p.in_size3; a.tile_cols = (int)p.in_size2;
    a.groups_per_tile = a.tile_rows / ce;
    const int64_t outer_rows = to ? p.in_size1 : p.in_size0;
    const int64_t outer_cols = to ? p.in_size0 : p.in_size1;
    a.row_groups = outer_rows * a.groups_per_tile;
    a.padded_cols = outer_cols * a.tile_cols;
    a.t_stride_orow_bytes = (to ? tile_elems : p.in_stride0) * es;
    a.t_stride_ocol_bytes = (to ? p.in_stride0 : tile_elems) * es;
    a.by_tile_cols = make_fastdiv((uint32_t)a.tile_cols);
    a.by_groups = make_fastdiv((uint32_t)a.groups_per_tile);
    a.padding = 0;
    a.blocks_x = a.blocks_y = 0;
    int st = es == 2 ? launch_unpack_transpose<2>(a, s) : launch_unpack_transpose<4>(a, s);
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
