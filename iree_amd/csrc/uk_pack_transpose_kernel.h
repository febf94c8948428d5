// The pack / unpack kernels for transposed inner tiles, as device functions:
// wrapped in a __global__ by the library (uk_pack.hip) and by the code object
// built for a HAL executable.
#ifndef IREE_AMD_UK_PACK_TRANSPOSE_KERNEL_H_
#define IREE_AMD_UK_PACK_TRANSPOSE_KERNEL_H_

#include "uk_pack_stream_kernel.h"

namespace uk {
namespace {

// n / d for 0 <= n < 2^31 and a fixed d >= 1: (n * mul) >> shift.
struct FastDiv {
  uint32_t mul, shift, d;
  __device__ __forceinline__ uint32_t div(uint32_t n) const {
    return d == 1 ? n : (uint32_t)(((uint64_t)n * mul) >> shift);
  }
};
__host__ __device__ inline FastDiv make_fastdiv(uint32_t d) {
  FastDiv f;
  f.d = d;
  uint32_t l = 0;
  while ((1ull << l) < d) ++l;
  f.shift = 31 + l;
  f.mul = (uint32_t)(((1ull << f.shift) + d - 1) / d);  // < 2^32 for d >= 2
  return f;
}

//---------------------------------------------------------------------------
// Pack with transposed inner tiles (the right-hand side of a matmul given as
// B[K][N]: every tile is stored column by column). A 16-byte chunk of the tiled
// buffer is then CE = 16/ES consecutive matrix ROWS of one matrix column. One
// thread builds one such chunk from CE element-sized loads and stores it with
// one 128-bit store. Lanes of a wave take 64 consecutive matrix columns, so
// every load instruction reads 64 consecutive elements of a row and the stores
// of a wave are whole tiles (or whole rows of chunks of a tile); a wave walks
// kTransUnroll consecutive row groups so that enough loads are in flight.
//---------------------------------------------------------------------------
constexpr int kTransUnroll = 4;

struct TransArgs {
  const char* mat;
  char* tiled;
  int64_t m_size0, m_size1, m_pitch_bytes;
  int64_t row_groups;            // outer_rows * groups_per_tile
  int64_t padded_cols;           // outer_cols * tile_cols
  int64_t t_stride_orow_bytes, t_stride_ocol_bytes;
  int tile_rows, tile_cols;      // matrix orientation: tile_rows = stored inner size
  int groups_per_tile;           // tile_rows / CE
  FastDiv by_tile_cols, by_groups;
  uint32_t blocks_x, blocks_y;
  uint64_t padding;
};

template <int ES>
__device__ __forceinline__ void pack_transpose_body(const TransArgs& a) {
  constexpr int CE = 16 / ES;
  typedef typename Chunk<ES>::elem_t elem_t;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // Same XCD-compact block order as the streaming kernels.
  uint32_t bx, by;
  {
    constexpr uint32_t kXcds = 8;
    const uint32_t total = a.blocks_x * a.blocks_y;
    const uint32_t per = total / kXcds, rem = total % kXcds;
    const uint32_t xcd = blockIdx.x % kXcds, idx = blockIdx.x / kXcds;
    const uint32_t logical = xcd * per + (xcd < rem ? xcd : rem) + idx;
    by = logical / a.blocks_x;
    bx = logical - by * a.blocks_x;
  }
  const int64_t c = (int64_t)bx * 64 + lane;                 // matrix column
  const int64_t g0 = ((int64_t)by * 4 + wave) * kTransUnroll;  // first row group of this wave
  if (g0 >= a.row_groups) return;
  const bool col_in_tiles = c < a.padded_cols;
  // where column c lands: tile column and row of the (transposed) tile
  const uint32_t cc = col_in_tiles ? (uint32_t)c : 0;
  const uint32_t ocol = a.by_tile_cols.div(cc), d2 = cc - ocol * a.tile_cols;
  char* out_col = a.tiled + (int64_t)ocol * a.t_stride_ocol_bytes + (int64_t)d2 * a.tile_rows * ES;
  const elem_t pad = (elem_t)a.padding;
  const bool interior = (int64_t)(bx + 1) * 64 <= a.m_size1 &&
                        (g0 + kTransUnroll) * CE <= a.m_size0 && g0 + kTransUnroll <= a.row_groups;
  elem_t v[kTransUnroll][CE];
  if (interior) {
    const char* src = a.mat + g0 * CE * a.m_pitch_bytes + c * ES;
#pragma unroll
    for (int u = 0; u < kTransUnroll; ++u)
#pragma unroll
      for (int i = 0; i < CE; ++i) v[u][i] = *(const elem_t*)(src + (int64_t)(u * CE + i) * a.m_pitch_bytes);
  } else {
#pragma unroll
    for (int u = 0; u < kTransUnroll; ++u)
#pragma unroll
      for (int i = 0; i < CE; ++i) {
        const int64_t r = (g0 + u) * CE + i;
        v[u][i] = (r < a.m_size0 && c < a.m_size1) ? *(const elem_t*)(a.mat + r * a.m_pitch_bytes + c * ES) : pad;
      }
  }
  if (!col_in_tiles) return;
#pragma unroll
  for (int u = 0; u < kTransUnroll; ++u) {
    const int64_t g = g0 + u;
    if (g >= a.row_groups) break;
    int64_t orow;
    uint32_t grp;
    if (g < 0x7FFFFFFF) {
      orow = a.by_groups.div((uint32_t)g);
      grp = (uint32_t)g - (uint32_t)orow * a.groups_per_tile;
    } else {
      orow = g / a.groups_per_tile;
      grp = (uint32_t)(g - orow * a.groups_per_tile);
    }
    union { elem_t e[CE]; u32x4 vec; } chunk;
#pragma unroll
    for (int i = 0; i < CE; ++i) chunk.e[i] = v[u][i];
    *(u32x4*)(out_col + orow * a.t_stride_orow_bytes + (int64_t)grp * 16) = chunk.vec;
  }
}

// The same for 1- and 2-byte elements with dword loads: a thread takes W = 4 / ES
// adjacent columns (one dword of every row) and builds W chunks, so that a
// wave's load instruction reads 256 bytes of a row instead of 64 or 128. The
// kernel above is bound by the rate at which a compute unit takes load
// instructions (f16 4096 x 4096 into 32x8 tiles: 17.2 -> 15.8 us). Needs rows
// that start on 4-byte boundaries and tiles of whole W columns (the host
// checks); a wave covers 64 W columns.
template <int ES>
__device__ __forceinline__ void pack_transpose_wide_body(const TransArgs& a) {
  static_assert(ES == 1 || ES == 2, "32-bit elements are dwords already");
  constexpr int CE = 16 / ES, W = 4 / ES;
  typedef typename Chunk<ES>::elem_t elem_t;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  uint32_t bx, by;
  {
    constexpr uint32_t kXcds = 8;
    const uint32_t total = a.blocks_x * a.blocks_y;
    const uint32_t per = total / kXcds, rem = total % kXcds;
    const uint32_t xcd = blockIdx.x % kXcds, idx = blockIdx.x / kXcds;
    const uint32_t logical = xcd * per + (xcd < rem ? xcd : rem) + idx;
    by = logical / a.blocks_x;
    bx = logical - by * a.blocks_x;
  }
  const int64_t c = ((int64_t)bx * 64 + lane) * W;           // first of this thread's columns
  const int64_t g0 = ((int64_t)by * 4 + wave) * kTransUnroll;  // first row group of this wave
  if (g0 >= a.row_groups) return;
  const bool col_in_tiles = c < a.padded_cols;   // (tiles are whole W columns: all of them or none)
  const uint32_t cc = col_in_tiles ? (uint32_t)c : 0;
  const uint32_t ocol = a.by_tile_cols.div(cc), d2 = cc - ocol * a.tile_cols;
  char* out_col = a.tiled + (int64_t)ocol * a.t_stride_ocol_bytes + (int64_t)d2 * a.tile_rows * ES;
  const uint32_t pad = (uint32_t)(elem_t)a.padding;
  const bool interior = (int64_t)(bx + 1) * 64 * W <= a.m_size1 &&
                        (g0 + kTransUnroll) * CE <= a.m_size0 && g0 + kTransUnroll <= a.row_groups;
  uint32_t v[kTransUnroll][CE];     // the W elements of one row, first column in the low bits
  if (interior) {
    const char* src = a.mat + g0 * CE * a.m_pitch_bytes + c * ES;
#pragma unroll
    for (int u = 0; u < kTransUnroll; ++u)
#pragma unroll
      for (int i = 0; i < CE; ++i) v[u][i] = *(const uint32_t*)(src + (int64_t)(u * CE + i) * a.m_pitch_bytes);
  } else {
#pragma unroll
    for (int u = 0; u < kTransUnroll; ++u)
#pragma unroll
      for (int i = 0; i < CE; ++i) {
        const int64_t r = (g0 + u) * CE + i;
        uint32_t d = 0;
#pragma unroll
        for (int w = 0; w < W; ++w) {
          const uint32_t e = (r < a.m_size0 && c + w < a.m_size1)
                                 ? (uint32_t)*(const elem_t*)(a.mat + r * a.m_pitch_bytes + (c + w) * ES) : pad;
          d |= e << (8 * ES * w);
        }
        v[u][i] = d;
      }
  }
  if (!col_in_tiles) return;
#pragma unroll
  for (int u = 0; u < kTransUnroll; ++u) {
    const int64_t g = g0 + u;
    if (g >= a.row_groups) break;
    int64_t orow;
    uint32_t grp;
    if (g < 0x7FFFFFFF) {
      orow = a.by_groups.div((uint32_t)g);
      grp = (uint32_t)g - (uint32_t)orow * a.groups_per_tile;
    } else {
      orow = g / a.groups_per_tile;
      grp = (uint32_t)(g - orow * a.groups_per_tile);
    }
    char* dst = out_col + orow * a.t_stride_orow_bytes + (int64_t)grp * 16;
#pragma unroll
    for (int w = 0; w < W; ++w) {
      union { elem_t e[CE]; u32x4 vec; } chunk;
#pragma unroll
      for (int i = 0; i < CE; ++i) chunk.e[i] = (elem_t)(v[u][i] >> (8 * ES * w));
      *(u32x4*)(dst + (int64_t)w * a.tile_rows * ES) = chunk.vec;
    }
  }
}

// 2-byte elements, whole rows of 16 bytes per lane: a wave covers 512 columns
// of the 8 matrix rows of one row group with 8 load instructions of 1 KiB each
// (the streaming pack's rate; the dword kernel above needs 32 for the same
// bytes). A lane then holds an 8 x 8 block, transposes it in registers (one
// byte permute per dword) into the 8 chunks of its 8 columns, and the wave
// passes the chunks through its 8 KiB of LDS so that store instruction s takes
// columns 64 s .. 64 s + 63, one per lane: 1 KiB of whole tiles per store where
// the lane's own 8 chunks would be 64 pieces of 16 bytes 128 bytes apart. LDS
// holds lane l's chunk w at 16-byte slot 8 l + (w + l / 2) mod 8: both the
// writes (lanes 128 bytes apart) and the reads (8 lanes per 128 bytes, two
// source lanes per 16) then touch every bank once per 16 lanes.
// kLdsUnroll row groups per wave, all loaded before the first is stored (4:
// 13.4 us for f16 4096 x 4096 into 32x8 tiles, 1: 14.3; the dword kernel 15.8).
template <int ES, int kLdsUnroll>
__device__ __forceinline__ void pack_transpose_lds_body(const TransArgs& a) {
  static_assert(ES == 2, "2-byte elements");
  typedef uint32_t u32x4u __attribute__((ext_vector_type(4), aligned(4)));
  __shared__ u32x4 exchange[4][512];
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  uint32_t bx, by;
  {
    constexpr uint32_t kXcds = 8;
    const uint32_t total = a.blocks_x * a.blocks_y;
    const uint32_t per = total / kXcds, rem = total % kXcds;
    const uint32_t xcd = blockIdx.x % kXcds, idx = blockIdx.x / kXcds;
    const uint32_t logical = xcd * per + (xcd < rem ? xcd : rem) + idx;
    by = logical / a.blocks_x;
    bx = logical - by * a.blocks_x;
  }
  const int64_t c0 = (int64_t)bx * 512;                       // first column of the wave
  const int64_t c = c0 + lane * 8;                            // first of this lane's 8 columns
  const int64_t g0 = ((int64_t)by * 4 + wave) * kLdsUnroll;   // first row group of this wave
  if (g0 >= a.row_groups) return;
  u32x4* xw = exchange[wave];
  const uint32_t pad = (uint16_t)a.padding;
  // all the loads of the wave's row groups first, so that they are in flight together
  u32x4 vall[kLdsUnroll][8];
  if (c0 + 512 <= a.m_size1 && (g0 + kLdsUnroll) * 8 <= a.m_size0) {
    const char* src = a.mat + g0 * 8 * a.m_pitch_bytes + c * 2;
#pragma unroll
    for (int u = 0; u < kLdsUnroll; ++u)
#pragma unroll
      for (int i = 0; i < 8; ++i) vall[u][i] = *(const u32x4u*)(src + (int64_t)(u * 8 + i) * a.m_pitch_bytes);
  } else {
#pragma unroll
    for (int u = 0; u < kLdsUnroll; ++u)
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int64_t r = (g0 + u) * 8 + i;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          uint32_t both = 0;
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const int64_t col = c + 2 * d + h;
            const uint32_t e = (r < a.m_size0 && col < a.m_size1)
                                   ? (uint32_t)*(const uint16_t*)(a.mat + r * a.m_pitch_bytes + col * 2) : pad;
            both |= e << (16 * h);
          }
          vall[u][i][d] = both;
        }
      }
  }
#pragma unroll
  for (int u = 0; u < kLdsUnroll; ++u) {
    const int64_t g = g0 + u;
    if (g >= a.row_groups) break;
    const u32x4 (&v)[8] = vall[u];
    // chunk w: column c + w, rows 0..7 of the group, row 2 j in the low half of dword j
#pragma unroll
    for (int w = 0; w < 8; ++w) {
      const uint32_t sel = (w & 1) ? 0x07060302u : 0x05040100u;
      u32x4 chunk;
#pragma unroll
      for (int j = 0; j < 4; ++j) chunk[j] = __builtin_amdgcn_perm(v[2 * j + 1][w / 2], v[2 * j][w / 2], sel);
      xw[lane * 8 + ((w + (lane >> 1)) & 7)] = chunk;
    }
    // (the wave's own LDS region: lanes run in lockstep and LDS serves a wave's
    // accesses in order; the fences keep the compiler from reordering them)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    int64_t orow;
    uint32_t grp;
    if (g < 0x7FFFFFFF) {
      orow = a.by_groups.div((uint32_t)g);
      grp = (uint32_t)g - (uint32_t)orow * a.groups_per_tile;
    } else {
      orow = g / a.groups_per_tile;
      grp = (uint32_t)(g - orow * a.groups_per_tile);
    }
    char* out_row = a.tiled + orow * a.t_stride_orow_bytes + (int64_t)grp * 16;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const uint32_t from = 8 * s + (lane >> 3);                 // the lane that built this chunk
      const u32x4 chunk = xw[from * 8 + (((lane & 7) + (from >> 1)) & 7)];
      const int64_t n = c0 + 64 * s + lane;
      if (n < a.padded_cols) {
        const uint32_t ocol = a.by_tile_cols.div((uint32_t)n), d2 = (uint32_t)n - ocol * a.tile_cols;
        *(u32x4*)(out_row + (int64_t)ocol * a.t_stride_ocol_bytes + (int64_t)d2 * a.tile_rows * 2) = chunk;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
}

// The reverse: unpack of tiles stored column by column (the transposed result
// tiles of a matmul whose narrow dimension was exchanged, reference
// unpack.c:190-247). One thread takes one 16-byte chunk of the tiled buffer
// (CE consecutive matrix rows of one column) and stores its CE elements; the
// lanes of a wave hold 64 consecutive columns, so every store instruction
// writes 64 consecutive elements of a matrix row. Same block walk as the pack.
template <int ES>
__device__ __forceinline__ void unpack_transpose_body(const TransArgs& a) {
  constexpr int CE = 16 / ES;
  typedef typename Chunk<ES>::elem_t elem_t;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  uint32_t bx, by;
  {
    constexpr uint32_t kXcds = 8;
    const uint32_t total = a.blocks_x * a.blocks_y;
    const uint32_t per = total / kXcds, rem = total % kXcds;
    const uint32_t xcd = blockIdx.x % kXcds, idx = blockIdx.x / kXcds;
    const uint32_t logical = xcd * per + (xcd < rem ? xcd : rem) + idx;
    by = logical / a.blocks_x;
    bx = logical - by * a.blocks_x;
  }
  const int64_t c = (int64_t)bx * 64 + lane;                 // matrix column
  const int64_t g0 = ((int64_t)by * 4 + wave) * kTransUnroll;  // first row group of this wave
  if (g0 >= a.row_groups || c >= a.m_size1 || c >= a.padded_cols) return;
  const uint32_t cc = (uint32_t)c;
  const uint32_t ocol = a.by_tile_cols.div(cc), d2 = cc - ocol * a.tile_cols;
  const char* in_col = a.tiled + (int64_t)ocol * a.t_stride_ocol_bytes + (int64_t)d2 * a.tile_rows * ES;
  union { elem_t e[CE]; u32x4 vec; } chunk[kTransUnroll];
#pragma unroll
  for (int u = 0; u < kTransUnroll; ++u) {
    const int64_t g = g0 + u;
    chunk[u].vec = u32x4{0u, 0u, 0u, 0u};
    if (g < a.row_groups) {
      int64_t orow;
      uint32_t grp;
      if (g < 0x7FFFFFFF) {
        orow = a.by_groups.div((uint32_t)g);
        grp = (uint32_t)g - (uint32_t)orow * a.groups_per_tile;
      } else {
        orow = g / a.groups_per_tile;
        grp = (uint32_t)(g - orow * a.groups_per_tile);
      }
      chunk[u].vec = *(const u32x4*)(in_col + orow * a.t_stride_orow_bytes + (int64_t)grp * 16);
    }
  }
  char* dst = (char*)a.mat + c * ES;
#pragma unroll
  for (int u = 0; u < kTransUnroll; ++u)
#pragma unroll
    for (int i = 0; i < CE; ++i) {
      const int64_t r = (g0 + u) * CE + i;
      if (r < a.m_size0) *(elem_t*)(dst + r * a.m_pitch_bytes) = chunk[u].e[i];
    }
}

// The same by blocks: a lane takes a CE x CE block of the matrix, i.e. the
// chunks of CE adjacent columns for one row group (CE loads of 16 bytes),
// transposes it in registers (32-bit elements: a renaming of registers;
// 16-bit ones: a byte permute per dword) and stores CE row pieces of 16 bytes.
// Lanes 0..15 of a wave hold 16 adjacent blocks of one row group, the four
// lane quarters four row groups: a load instruction reads, for 16 columns CE
// apart, the 64 contiguous bytes that four row groups of a stored column make
// (the kernel above: 64 pieces of 16 bytes, one per column), and a store
// instruction writes 256 contiguous bytes of each of 4 matrix rows (the
// kernel above: 64 elements of one row). One wave per workgroup, one quartet
// of row groups per wave (4 KiB of 32-bit, 8 KiB of 16-bit elements), waves
// that lie wholly inside the matrix as straight-line code. Needs tiles of
// whole CE columns (the host checks). Measured, f32 4096 x 4096 from 32x32
// tiles stored column by column: 31.7 us with the kernel above, 27.0 with
// this one; with two quartets per wave 31.0, as four waves per workgroup
// 32.9, non-temporal stores 27.9, ordinary loads 28.5. kLX = 8: 8 blocks
// across and 8 row groups per wave, for tiles of 8 row groups and more, whose
// stored columns are whole 128-byte lines that the wave then reads alone:
// 24.3 us (25.7 with non-temporal stores).
template <int ES, int kLX = 16, bool kNtStore = false>
__device__ __forceinline__ void unpack_transpose_block_body(const TransArgs& a) {
  // kLX blocks across and kGY = 64 / kLX row groups per wave
  constexpr int kU = 1, kWavesPerGroup = 1, kGY = 64 / kLX;
  constexpr bool kNtLoad = true;
  static_assert(ES == 2 || ES == 4, "results are 16- or 32-bit");
  constexpr int CE = 16 / ES;
  typedef typename Chunk<ES>::elem_t elem_t;
  typedef typename Chunk<ES>::aligned_t mat_vec_t;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  uint32_t bx, by;
  {
    constexpr uint32_t kXcds = 8;
    const uint32_t total = a.blocks_x * a.blocks_y;
    const uint32_t per = total / kXcds, rem = total % kXcds;
    const uint32_t xcd = blockIdx.x % kXcds, idx = blockIdx.x / kXcds;
    const uint32_t logical = xcd * per + (xcd < rem ? xcd : rem) + idx;
    by = logical / a.blocks_x;
    bx = logical - by * a.blocks_x;
  }
  const uint32_t lc = lane % kLX, lg = lane / kLX;
  const int64_t cols = a.m_size1 < a.padded_cols ? a.m_size1 : a.padded_cols;
  const int64_t c = ((int64_t)bx * kLX + lc) * CE;             // first of this lane's CE columns
  const int64_t g0 = ((int64_t)by * kWavesPerGroup + wave) * kGY * kU;   // first row group of this wave
  if (g0 >= a.row_groups || c >= cols) return;
  const uint32_t cc = (uint32_t)c;
  const uint32_t ocol = a.by_tile_cols.div(cc), d2 = cc - ocol * a.tile_cols;
  const char* in_col = a.tiled + (int64_t)ocol * a.t_stride_ocol_bytes + (int64_t)d2 * a.tile_rows * ES;
  const int64_t col_pitch = (int64_t)a.tile_rows * ES;         // between the stored columns of a tile
  const int n_cols = cols - c < CE ? (int)(cols - c) : CE;
  u32x4 v[kU][CE];
  char* dst = (char*)a.mat + c * ES;
  // One row of the lane's block as the 16 bytes to store.
  auto block_row = [&](const u32x4 (&blk)[CE], int i) -> u32x4 {
    if constexpr (ES == 4) {
      return u32x4{blk[0][i], blk[1][i], blk[2][i], blk[3][i]};
    } else {
      // row i of column j is half i % 2 of dword i / 2 of the column's chunk
      const uint32_t sel = (i & 1) ? 0x07060302u : 0x05040100u;
      u32x4 r;
#pragma unroll
      for (int e = 0; e < 4; ++e) r[e] = __builtin_amdgcn_perm(blk[2 * e + 1][i / 2], blk[2 * e][i / 2], sel);
      return r;
    }
  };
  auto source_of = [&](int64_t g) -> const char* {
    int64_t orow;
    uint32_t grp;
    if (g < 0x7FFFFFFF) {
      orow = a.by_groups.div((uint32_t)g);
      grp = (uint32_t)g - (uint32_t)orow * a.groups_per_tile;
    } else {
      orow = g / a.groups_per_tile;
      grp = (uint32_t)(g - orow * a.groups_per_tile);
    }
    return in_col + orow * a.t_stride_orow_bytes + (int64_t)grp * 16;
  };
  // Interior waves (all 16 blocks across lie inside the matrix, all row groups
  // exist and end inside it): straight-line code, every load issued before the
  // first store.
  const bool interior = ((int64_t)bx * kLX + kLX) * CE <= cols && g0 + kGY * kU <= a.row_groups &&
                        (g0 + kGY * kU) * CE <= a.m_size0;
  if (interior) {
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      const char* src = source_of(g0 + u * kGY + lg);
#pragma unroll
      for (int j = 0; j < CE; ++j)
        v[u][j] = kNtLoad ? __builtin_nontemporal_load((const u32x4*)(src + j * col_pitch)) : *(const u32x4*)(src + j * col_pitch);
    }
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      char* p = dst + (g0 + u * kGY + lg) * CE * a.m_pitch_bytes;
#pragma unroll
      for (int i = 0; i < CE; ++i) {
        if (kNtStore) __builtin_nontemporal_store((mat_vec_t)block_row(v[u], i), (mat_vec_t*)(p + i * a.m_pitch_bytes));
        else *(mat_vec_t*)(p + i * a.m_pitch_bytes) = block_row(v[u], i);
      }
    }
    return;
  }
#pragma unroll 1
  for (int u = 0; u < kU; ++u) {
    const int64_t g = g0 + u * kGY + lg;
    if (g >= a.row_groups) continue;
    const char* src = source_of(g);
#pragma unroll
    for (int j = 0; j < CE; ++j) v[0][j] = j < n_cols ? *(const u32x4*)(src + j * col_pitch) : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < CE; ++i) {
      const int64_t r = g * CE + i;
      if (r >= a.m_size0) continue;
      union { u32x4 vec; elem_t e[CE]; } row;
      row.vec = block_row(v[0], i);
      char* p = dst + r * a.m_pitch_bytes;
      if (n_cols == CE) {
        *(mat_vec_t*)p = row.vec;
      } else {
        for (int j = 0; j < n_cols; ++j) ((elem_t*)p)[j] = row.e[j];
      }
    }
  }
}

}  // namespace
}  // namespace uk

#endif  // IREE_AMD_UK_PACK_TRANSPOSE_KERNEL_H_
