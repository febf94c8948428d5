// The streaming pack / unpack kernel for power-of-two tiles, as a device
// function: wrapped in a __global__ by the library (uk_pack.hip) and by the code
// object built for a HAL executable.
#ifndef IREE_AMD_UK_PACK_STREAM_KERNEL_H_
#define IREE_AMD_UK_PACK_STREAM_KERNEL_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace uk {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// 128-bit access to memory that is only element-aligned.
template <int ES> struct Chunk;
template <> struct Chunk<1> { typedef u32x4 aligned_t __attribute__((aligned(1))); typedef uint8_t elem_t; };
template <> struct Chunk<2> { typedef u32x4 aligned_t __attribute__((aligned(2))); typedef uint16_t elem_t; };
template <> struct Chunk<4> { typedef u32x4 aligned_t __attribute__((aligned(4))); typedef uint32_t elem_t; };

constexpr int kStreamThreads = 256;
constexpr int kStreamUnroll = 2;

// The streaming kernels walk the MATRIX in blocks of R rows x 64 / R chunks
// per wave instruction: lane = (row in block) * (64 / R) + (chunk in block).
// On the matrix side every row segment is 1024 / R contiguous bytes; on the
// tiled side the R rows of one tile column are contiguous as well (R tile rows
// of cpr chunks each), so neither side moves less than a cache line at a time.
// The kernels for general tile geometry (uk_pack.hip) use R = 8 with
// kStreamUnroll vertically adjacent blocks per wave and 4 waves side by side:
constexpr int kBlockRows = 8, kBlockChunks = 8;
// The power-of-two kernel below takes its block shape as template parameters:
// kRowsPerBlock rows x 64 / kRowsPerBlock chunks per wave instruction, kUnroll
// vertically adjacent blocks per wave, kWaves waves per workgroup of which kWX
// side by side. Measured on MI355X (f16 8191 x 5001 <-> 32x16 tiles, TB/s,
// pack / unpack): 8 rows x 8 chunks, 2 blocks, 4 waves side by side 5.31 /
// 4.78; one block per wave 5.50 / 5.10; 4 rows x 16 chunks (256 bytes of a
// row), one block 5.50-5.54 / 5.24-5.30, as 2 x 2 waves 5.54 / 5.35, as one
// wave per workgroup 5.61 / 5.38 (the library's choice: the smallest unit of
// work, 4 KiB, scheduled on its own); 2 rows x 32 chunks 4.82 / 4.78; 16 rows
// x 4 chunks 5.42 / 4.87; more blocks per wave lose in every shape. Longer row
// pieces halve the partly written cache lines of ragged rows, which is what
// unpack gains from.
constexpr int kPow2Rows = 4, kPow2Unroll = 1, kPow2WavesX = 1, kPow2Waves = 1;

// Power-of-two tile geometry (every gfx950 tile shape): the same 8x8 block walk
// with all 64-bit address arithmetic done once per wave on the scalar unit and
// only 32-bit offsets per lane. kPack selects the direction.
struct Pow2Args {
  const char* mat;
  char* tiled;
  int64_t m_size0, m_size1;             // elements
  int64_t m_pitch_bytes;
  int64_t t_stride_row_bytes, t_stride_col_bytes;
  int64_t padded_rows;
  uint32_t chunks_per_row, padded_chunks_per_row;
  int log2_tile_rows, log2_cpr;
  uint32_t blocks_x, blocks_y;   // logical grid; launched as blocks_x * blocks_y workgroups
  uint64_t padding;
};

// Non-temporal accesses (measured on MI355X, f16 8191 x 5001 <-> 32x16 tiles).
// The tiled side's pieces are whole runs that nobody else touches: streaming
// them past the caches always pays (pack stores, unpack loads). On the matrix
// side it depends on the length of the row pieces. With 256-byte pieces (the
// library's block shape) non-temporal LOADS pay too (pack 5.65 -> 5.82 TB/s),
// non-temporal STORES still lose (unpack 5.41 -> 5.22: pieces of DRAM pages
// that are no longer merged); with the earlier 128-byte pieces, which share
// both their cache lines with neighbouring waves, the loads lost as well (pack
// 5.25 -> 4.5) and the stores were ruinous (unpack 4.76 -> 3.0). A plain copy
// with 8 KiB runs on both sides reaches 5.3-5.5 TB/s with ordinary and 6.0-6.4
// with non-temporal accesses on the same machine. Staging 32 rows x 1 KiB per
// workgroup through LDS, so that every wave instruction moves 1 KiB of one
// matrix row or of consecutive tile memory, was slower in all four
// combinations of non-temporal sides (pack 4.4-5.0, unpack 4.2-4.5 TB/s):
// longer runs per instruction do not pay for the barrier and the fewer, larger
// workgroups.
template <int ES, bool kPack, bool kNtLoad = true, bool kNtStore = kPack, int kBlockRows = kPow2Rows,
          int kStreamUnroll = kPow2Unroll, int kWX = kPow2WavesX, int kWaves = kPow2Waves>
__device__ __forceinline__ void stream_pow2_body(const Pow2Args a) {
  constexpr int CE = 16 / ES;
  constexpr int kBlockChunks = 64 / kBlockRows;
  constexpr int kRows = kBlockRows * kStreamUnroll;
  typedef typename Chunk<ES>::aligned_t mat_vec_t;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // Workgroup ids go round-robin over the 8 XCDs, each with its own L2. Give
  // XCD x the x-th contiguous slice of the row-major block sequence, so that
  // blocks that share a cache line (rows are rarely line-aligned) meet in one L2.
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
  const uint32_t j0 = (bx * kWX + wave % kWX) * kBlockChunks;
  const uint32_t col_limit = kPack ? a.padded_chunks_per_row : a.chunks_per_row;
  if (j0 >= col_limit) return;
  const int64_t row_limit = kPack ? a.padded_rows : a.m_size0;
  const int64_t r0 = ((int64_t)by * (kWaves / kWX) + wave / kWX) * kRows;
  if (r0 >= row_limit) return;
  const uint32_t tile_rows = 1u << a.log2_tile_rows, cpr = 1u << a.log2_cpr;
  const uint32_t jl = lane % kBlockChunks, rl = lane / kBlockChunks;
  // Scalar bases of this wave's block on both sides.
  const char* mat_base = a.mat + r0 * a.m_pitch_bytes + (int64_t)j0 * 16;
  char* tiled_base = a.tiled + (r0 >> a.log2_tile_rows) * a.t_stride_row_bytes +
                     (int64_t)(j0 >> a.log2_cpr) * a.t_stride_col_bytes;
  const uint32_t trow0 = (uint32_t)r0 & (tile_rows - 1), h0 = j0 & (cpr - 1);
  // Per-lane 32-bit offsets.
  const uint32_t pitch = (uint32_t)a.m_pitch_bytes;
  const uint32_t srow = (uint32_t)a.t_stride_row_bytes, scol = (uint32_t)a.t_stride_col_bytes;
  uint32_t mat_off[kStreamUnroll], tiled_off[kStreamUnroll];
#pragma unroll
  for (int u = 0; u < kStreamUnroll; ++u) {
    const uint32_t r = trow0 + u * kBlockRows + rl, j = h0 + jl;
    mat_off[u] = (u * kBlockRows + rl) * pitch + jl * 16;
    tiled_off[u] = (r >> a.log2_tile_rows) * srow + (j >> a.log2_cpr) * scol +
                   (((r & (tile_rows - 1)) << a.log2_cpr) + (j & (cpr - 1))) * 16;
  }
  const bool interior = (int64_t)(j0 + kBlockChunks) * CE <= a.m_size1 && r0 + kRows <= a.m_size0;
  if (interior) {
    u32x4 v[kStreamUnroll];
#pragma unroll
    for (int u = 0; u < kStreamUnroll; ++u) {
      if (kPack) {
        const mat_vec_t* p = (const mat_vec_t*)(mat_base + mat_off[u]);
        v[u] = kNtLoad ? __builtin_nontemporal_load(p) : *p;
      } else {
        const u32x4* p = (const u32x4*)(tiled_base + tiled_off[u]);
        v[u] = kNtLoad ? __builtin_nontemporal_load(p) : *p;
      }
    }
#pragma unroll
    for (int u = 0; u < kStreamUnroll; ++u) {
      if (kPack) {
        u32x4* p = (u32x4*)(tiled_base + tiled_off[u]);
        if (kNtStore) __builtin_nontemporal_store(v[u], p); else *p = v[u];
      } else {
        mat_vec_t* p = (mat_vec_t*)((char*)mat_base + mat_off[u]);
        if (kNtStore) __builtin_nontemporal_store((mat_vec_t)v[u], p); else *p = v[u];
      }
    }
    return;
  }
  // Edge blocks: per-lane predicates, padding (pack), byte-wise handling of the
  // chunk that straddles the right edge.
  if (j0 + jl >= col_limit) return;
  const int64_t c = (int64_t)(j0 + jl) * CE;
  u32x4 pad_vec;
  {
    uint64_t p = a.padding;
    if (ES == 1) { p &= 0xFF; p |= p << 8; p |= p << 16; p |= p << 32; }
    if (ES == 2) { p &= 0xFFFF; p |= p << 16; p |= p << 32; }
    if (ES == 4) { p &= 0xFFFFFFFFull; p |= p << 32; }
    pad_vec = u32x4{(uint32_t)p, (uint32_t)(p >> 32), (uint32_t)p, (uint32_t)(p >> 32)};
  }
#pragma unroll 1
  for (int u = 0; u < kStreamUnroll; ++u) {
    const int64_t r = r0 + u * kBlockRows + rl;
    if (r >= row_limit) continue;
    const bool in_matrix = r < a.m_size0 && c < a.m_size1;
    const int valid = in_matrix ? (c + CE <= a.m_size1 ? 16 : (int)(a.m_size1 - c) * ES) : 0;
    union { u32x4 vec; uint8_t b[16]; } tmp;
    if (kPack) {
      tmp.vec = pad_vec;
      if (valid == 16) tmp.vec = *(const mat_vec_t*)(mat_base + mat_off[u]);
      else for (int i = 0; i < valid; ++i) tmp.b[i] = ((const uint8_t*)(mat_base + mat_off[u]))[i];
      *(u32x4*)(tiled_base + tiled_off[u]) = tmp.vec;
    } else {
      tmp.vec = *(const u32x4*)(tiled_base + tiled_off[u]);
      if (valid == 16) *(mat_vec_t*)((char*)mat_base + mat_off[u]) = tmp.vec;
      else for (int i = 0; i < valid; ++i) ((uint8_t*)mat_base + mat_off[u])[i] = tmp.b[i];
    }
  }
}

}  // namespace
}  // namespace uk

#endif  // IREE_AMD_UK_PACK_STREAM_KERNEL_H_
