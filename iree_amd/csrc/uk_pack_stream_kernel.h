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

// Unpack whose stores are whole, aligned cache lines. The rows of a matrix
// rarely start on a 128-byte line (8191 x 5001 f16: every row starts 10002
// bytes after the one before), so a kernel that moves 16-byte chunks from
// their place in a tile to their place in the row writes pieces that begin and
// end inside lines it shares with the neighbouring pieces, and non-temporal
// stores of such pieces lose (measured with the kernel above: 5.40 TB/s with
// ordinary stores, 5.26 with non-temporal ones; on a matrix whose rows do
// start on lines 5.61 and 5.94). Here a wave instead owns, for each of 4
// rows, one 256-byte window of MEMORY that starts on a line: lane (row, t)
// produces the 16 bytes at window + 16 t, which are bytes o .. o + 16 of the
// row for an o that is rarely a multiple of 16. It loads the tile chunk o / 16,
// takes the next one from the next lane (a cross-lane move; the last lane of a
// row loads its own), shifts the pair right by o % 16 bytes (a dword select by
// two bits of the shift and a byte align by the other two) and stores 16
// aligned bytes non-temporally. Only the first and last window of a row write
// partial chunks, element by element. Same tile geometry as the kernel above
// (power-of-two tiles, no inner transpose). Measured: 8191 x 5001 f16 from
// 32x16 tiles 5.78 TB/s (5.40 with the kernel above), 8192 x 5120 6.05; two
// and four blocks of rows per wave 5.32 and 4.99; loading both chunks per
// lane 3.7 (non-temporal: the shared chunk comes from memory twice) to 4.1.
template <int ES, int kU = 1>
__device__ __forceinline__ void unpack_aligned_body(const Pow2Args a) {
  typedef typename Chunk<ES>::elem_t elem_t;
  constexpr int CE = 16 / ES;
  const uint32_t lane = threadIdx.x & 63;
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
  // All 64-bit arithmetic is the wave's (scalar unit); lanes work with 32-bit
  // offsets from the wave's first row on both sides.
  const int64_t r0 = (int64_t)by * (4 * kU);
  const char* mat_base = a.mat + r0 * a.m_pitch_bytes;
  const char* tiled_base = a.tiled + (r0 >> a.log2_tile_rows) * a.t_stride_row_bytes;
  const uint32_t rows_left = (uint32_t)(a.m_size0 - r0 < 4 * kU ? a.m_size0 - r0 : 4 * kU);
  const uint32_t mat_lo = (uint32_t)(uintptr_t)mat_base;
  const uint32_t pitch = (uint32_t)a.m_pitch_bytes;
  const uint32_t srow = (uint32_t)a.t_stride_row_bytes, scol = (uint32_t)a.t_stride_col_bytes;
  const uint32_t tile_rows = 1u << a.log2_tile_rows, cpr = 1u << a.log2_cpr;
  const uint32_t trow0 = (uint32_t)r0 & (tile_rows - 1);
  const int32_t row_bytes = (int32_t)(a.m_size1 * ES);
  const int32_t last_chunk = (int32_t)a.padded_chunks_per_row - 1;
  const uint32_t rl = lane >> 4, t = lane & 15;
  u32x4 lo[kU], hi[kU];
  int32_t o[kU];
  uint32_t row_off[kU];
  bool row_ok[kU];
  // all the loads of the wave's kU blocks of 4 rows first
#pragma unroll
  for (int u = 0; u < kU; ++u) {
    const uint32_t rloc = u * 4 + rl;
    row_ok[u] = rloc < rows_left;
    const uint32_t rr = row_ok[u] ? rloc : rows_left - 1;    // (loads of a row past the end stay inside the buffer)
    row_off[u] = rr * pitch;
    // this lane's 16 bytes of memory (bx-th window of the row's first line on) and where in the row they lie
    const uint32_t head = (mat_lo + row_off[u]) & 127u;
    o[u] = (int32_t)(bx * 256 + t * 16) - (int32_t)head;     // -127 ..
    const int32_t q = o[u] >> 4;                             // (floor)
    const uint32_t r = trow0 + rr;
    const uint32_t in_panel = (r >> a.log2_tile_rows) * srow + ((r & (tile_rows - 1)) << a.log2_cpr) * 16;
    auto chunk_at = [&](int32_t qq) -> const u32x4* {
      qq = qq < 0 ? 0 : (qq > last_chunk ? last_chunk : qq);
      return (const u32x4*)(tiled_base + (in_panel + ((uint32_t)qq >> a.log2_cpr) * scol + ((uint32_t)qq & (cpr - 1)) * 16));
    };
    // The second chunk is the first one of the next lane of the row (fetched
    // from there across lanes; loading it as well doubled the reads); the
    // row's last lane loads its own.
    lo[u] = __builtin_nontemporal_load(chunk_at(q));
    hi[u] = u32x4{0u, 0u, 0u, 0u};
    if (t == 15 && (o[u] & 15)) hi[u] = *chunk_at(q + 1);
  }
#pragma unroll
  for (int u = 0; u < kU; ++u) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      // (row_shl:1: lane t of a row of 16 takes lane t + 1's value, lane 15 keeps its own)
      hi[u][i] = (uint32_t)__builtin_amdgcn_update_dpp((int)hi[u][i], (int)lo[u][i], 0x101, 0xf, 0xf, false);
    }
  }
#pragma unroll
  for (int u = 0; u < kU; ++u) {
    // bytes sb .. sb + 16 of lo : hi (everything in named registers: an array
    // here ends up in LDS)
    const uint32_t sb = (uint32_t)o[u] & 15;
    const bool by8 = (sb & 8) != 0, by4 = (sb & 4) != 0;
    const uint32_t a0 = by8 ? lo[u].z : lo[u].x, a1 = by8 ? lo[u].w : lo[u].y, a2 = by8 ? hi[u].x : lo[u].z,
                   a3 = by8 ? hi[u].y : lo[u].w, a4 = by8 ? hi[u].z : hi[u].x, a5 = by8 ? hi[u].w : hi[u].y;
    const uint32_t b0 = by4 ? a1 : a0, b1 = by4 ? a2 : a1, b2 = by4 ? a3 : a2, b3 = by4 ? a4 : a3, b4 = by4 ? a5 : a4;
    u32x4 out;
    out.x = __builtin_amdgcn_alignbyte(b1, b0, sb & 3);
    out.y = __builtin_amdgcn_alignbyte(b2, b1, sb & 3);
    out.z = __builtin_amdgcn_alignbyte(b3, b2, sb & 3);
    out.w = __builtin_amdgcn_alignbyte(b4, b3, sb & 3);
    if (!row_ok[u]) continue;
    char* dst = (char*)mat_base + row_off[u] + o[u];
    if (o[u] >= 0 && o[u] + 16 <= row_bytes) {
      __builtin_nontemporal_store(out, (u32x4*)dst);
    } else if (o[u] + 16 > 0 && o[u] < row_bytes) {
      // (row start and row end are whole elements, and so is every piece of a chunk)
#pragma unroll
      for (int e = 0; e < CE; ++e) {
        const int32_t at = o[u] + e * ES;
        const uint32_t word = e * ES / 4 == 0 ? out.x : e * ES / 4 == 1 ? out.y : e * ES / 4 == 2 ? out.z : out.w;
        if (at >= 0 && at < row_bytes) ((elem_t*)dst)[e] = (elem_t)(word >> (8 * (e * ES % 4)));
      }
    }
  }
}

}  // namespace
}  // namespace uk

#endif  // IREE_AMD_UK_PACK_STREAM_KERNEL_H_
