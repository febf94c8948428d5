// The mmt4d, pack and unpack kernels as a gfx950 code object for a HAL
// executable on a HIP device: the device-resident route of the reference, where hand-written
// kernels are linked into a `hal.executable.source` through
// `#hal.executable.object<{path = "...co"}>`
// (samples/custom_dispatch/hip/kernels/example.mlir:36-118) and launched by the
// HIP HAL driver (runtime/src/iree/hal/drivers/hip/stream_command_buffer.c:519-581).
//
// ABI of every kernel here, as that driver packs it (kernels.cu:16-23 of the
// same sample): C name, the binding device pointers in order, then one 32-bit
// push constant per kernel parameter:
//
//   bindings        0 lhs (read only), 1 rhs (read only), 2 out
//   push constants  M, N, K   outer tile counts, as iree_uk_mmt4d takes them
//                             (runtime/src/iree/builtins/ukernel/mmt4d.h:14-21)
//                   K0        elements per tile row (M0 = N0 = 32)
//                   flags     the ukernel's flag word; IREE_UK_FLAG_MMT4D_ACCUMULATE
//                             (0x100, exported_bits.h:43) is the one bit read here,
//                             the type is fixed by the kernel's name
//   (mi355x_mmt4d_unpack_*: two more, out_rows and out_cols)
//
// Operands are dense: lhs is [M][K][32][K0], rhs [N][K][32][K0], out
// [M][N][32][32] (mi355x_mmt4d_unpack_*: the row-major out_rows x out_cols matrix
// an unpack of it would give; accumulates from there as well). K >= 1, every
// binding 16-byte aligned.
//
// Launch shape, fixed per export (workgroup_size and workgroup_local_memory of
// the hal.executable.export): 256 threads; the dynamic LDS size and the macro
// tile T (outer tiles of 32 rows per workgroup, both ways) are those of the
// table at the end of this file. The grid is ceildiv(M, T) * ceildiv(N, T)
// workgroups in x; in y it is 1, or the batch count of a linalg.batch_mmt4d:
// workgroup plane y works on the y-th of `batch` dense problems laid one after
// the other in each binding ([batch][M][K][32][K0] and so on; the row-major
// result of mi355x_mmt4d_unpack_* is [batch][out_rows][out_cols]).
//
// mi355x_matmul_packed_rhs_*: the whole linear layer out[M][N] (+)= lhs[M][K] *
// rhs in one dispatch: bindings 0 lhs, the dense row-major M x K matrix (read
// only), 1 rhs, packed [ceildiv(N, 32)][K / K0][32][K0] (read only: weights
// packed ahead of time), 2 out, the dense row-major M x N matrix; push
// constants M, N, K (ELEMENTS; K a whole number of matrix-core K-steps: 32 for
// f16 / bf16 / i8, 8 for f32, 64 for fp8 and the s8s8s32_k64 exports, which
// take K0 = 16 only and are the faster i8 form), K0, flags. Macro tiles of 128 x 256
// (_t4x8: the cheaper one for a row-major left-hand side, two workgroups per
// compute unit) or 256 x 256 (_t8x8); grid = ceildiv(ceildiv(M, 32), 4 or 8) *
// ceildiv(ceildiv(N, 32), 8).
//
// mi355x_pack_{8,16,32}bit / mi355x_unpack_{16,32}bit: iree_uk_pack / iree_uk_unpack
// without transposes (runtime/src/iree/builtins/ukernel/pack.h:26-34,
// unpack.h:17-25) on dense operands, for power-of-two tiles whose rows are whole
// 16-byte chunks:
//
//   pack    bindings 0 in: the size0 x size1 matrix (read only), 1 out: tiles
//           [ceildiv(size0, tile0)][ceildiv(size1, tile1)][tile0][tile1]
//           push constants size0, size1, tile0, tile1, padding (the element's bits)
//   unpack  bindings 0 in: the tiles (read only), 1 out: the size0 x size1 matrix
//           push constants size0, size1, tile0, tile1
//
// mi355x_pack_transpose_{8,16,32}bit / mi355x_unpack_transpose_{16,32}bit: the same
// with transposed inner tiles (IREE_UK_FLAG_PACK_TRANSPOSE_INNER, pack.c:131-166,
// unpack.c:190-247: what the right-hand side B[K][N] of a matmul needs, and
// the transposed result tiles of a narrow-N matmul): a tile covers tile0 rows
// x tile1 columns of the matrix and is stored column by column,
// [ceildiv(size0, tile0)][ceildiv(size1, tile1)][tile1][tile0]; same bindings
// and push constants; power-of-two tiles with tile0 * bytes >= 16; grid =
// ceildiv(C, 64) * ceildiv(G, 16) with G = ceildiv(size0, tile0) * tile0 * bytes
// / 16 (groups of rows that make one 16-byte chunk) and C = the padded columns
// ceildiv(size1, tile1) * tile1 (pack) or size1 (unpack).
//
// mi355x_dequant_matmul_i4_k4096_g128_{r16,r32}: the grouped int4-weight
// dequantising matmul of the decode step (the dispatch
// compiler/src/iree/compiler/GlobalOptimization/FuseDequantizationMatmul.cpp:53-159
// forms; no ukernel in the reference): out[M][N] f16 = x[M][4096] f16 times
// weights of N columns in groups of 128 along K with f16 scales and packed
// uint4 zero points. Bindings 0 x, 1 the weights in the library's tiled layout
// (iree_amd_uk_pack_i4_weights), 2 scales [N][32] f16, 3 zero points [N][32]
// packed two to a byte (all read only), 4 out; push constants M, N. N a
// multiple of 32; _r16 takes 1..16 rows, _r32 1..32 (anything else writes
// nothing). 512 threads, 128 KiB of dynamic LDS (plus 32 KiB static in _r16),
// grid = min(N / 32, 256).
//
// 256 threads, no LDS; grid = ceildiv(C, 32) * ceildiv(R, 16) with, for pack,
// C = ceildiv(size1, tile1) * tile1 * bytes / 16 and R = ceildiv(size0, tile0) *
// tile0 (the padded extent), for unpack C = ceildiv(size1 * bytes, 16) and
// R = size0. Limits (32-bit offsets inside a block of 16 rows): a matrix row
// and one outer row of tiles below 2^26 bytes each.
#include "../csrc/uk_mmt4d_mfma_kernel.h"
#include "../csrc/uk_pack_stream_kernel.h"
#include "../csrc/uk_pack_transpose_kernel.h"
#include "../csrc/uk_i4_kernel.h"

namespace {

using namespace uk;

template <typename Cfg, int WM, int WN, int kRing, int kSync, bool row_major>
__device__ __forceinline__ void hal_mmt4d(const void* lhs, const void* rhs, void* out, int M, int N,
                                          int K, int K0, uint32_t flags, int out_rows, int out_cols) {
  constexpr int kPerTile = 32 / Cfg::kRows;
  constexpr int TM = 2 * WM, TN = 2 * WN;
  static_assert(TM == TN && TM % kPerTile == 0, "square macro tile of whole outer tiles");
  typedef typename Cfg::out_t out_t;
  MfmaArgs a;
  const int64_t k_elems = (int64_t)K * K0;
  a.lhs = (const char*)lhs;
  a.rhs = (const char*)rhs;
  a.out = (char*)out;
  a.lhs_stride_bytes = a.rhs_stride_bytes = k_elems * 32 * Cfg::kElemBytes;
  a.out_stride_bytes = row_major ? (int64_t)out_cols * (int64_t)sizeof(out_t)
                                 : (int64_t)N * 1024 * (int64_t)sizeof(out_t);
  a.M = M;
  a.N = N;
  a.panel_rows = 4;
  a.ksteps = (int)(k_elems / Cfg::kMfmaK);
  a.tail_tiles = (int)((k_elems % Cfg::kMfmaK) / K0);
  a.tiles_m = (M * kPerTile + TM - 1) / TM;
  a.tiles_n = (N * kPerTile + TN - 1) / TN;
  a.accumulate = (flags & 0x100u) != 0;
  a.row_major_out = row_major;
  a.out_rows = out_rows;
  a.out_cols = out_cols;
  a.lhs_row_major = 0;
  a.k_slices = 0; a.batch = 1; a.batch_by_xcd = 0;
  a.stream_out = (int64_t)M * N * 1024 * (int64_t)sizeof(out_t) > (32ll << 20);
  a.slice_ksteps = 0;
  a.slice_out_bytes = 0;
  a.k0_div = Cfg::kMfmaK / K0;
  a.gate_scale = a.up_scale = a.inv_out_scale = a.out_scale = 1.0f;
  if (K < 1) return;
  // Batch entry blockIdx.y of dense operands. Workgroups go to the 8 XCDs
  // round-robin in launch order; entries of at most 64 macro tiles are dealt to
  // the XCDs whole (the leading multiple of 8 planes: workgroup L takes tile
  // (L / 8) % tiles of plane L % 8 + 8 * (L / 8 / tiles)), so that the tiles of
  // an entry share their operands in one L2.
  unsigned plane_y = blockIdx.y, bid = blockIdx.x;
  if (gridDim.x <= 64 && blockIdx.y < gridDim.y / 8 * 8) {
    const unsigned linear = blockIdx.y * gridDim.x + blockIdx.x;
    const unsigned j = linear / 8;
    plane_y = linear % 8 + 8 * (j / gridDim.x);
    bid = j % gridDim.x;
  }
  // a grid larger than the tile count (a count region that rounds up) is harmless
  if ((int)bid >= a.tiles_m * a.tiles_n) return;
  const int64_t plane = plane_y;
  a.lhs += plane * M * a.lhs_stride_bytes;
  a.rhs += plane * N * a.rhs_stride_bytes;
  a.out += plane * (row_major ? out_rows : M) * a.out_stride_bytes;
  mmt4d_mfma_body<Cfg, WM, WN, kRing, kSync, false, 2, row_major ? 1 : 0>(a, (int)bid);
}

template <typename Cfg, int WM, int WN, int kRing, int kSync>
__device__ __forceinline__ void hal_matmul_packed_rhs(const void* lhs, const void* rhs, void* out,
                                                      int M, int N, int K, int K0, uint32_t flags) {
  constexpr int kPerTile = 32 / Cfg::kRows;
  constexpr int TM = 2 * WM, TN = 2 * WN;
  static_assert(TM % kPerTile == 0 && TN % kPerTile == 0, "macro tile of whole outer tiles");
  typedef typename Cfg::out_t out_t;
  if (M < 1 || N < 1 || K < Cfg::kMfmaK || K % Cfg::kMfmaK) return;
  if (Cfg::kSub == 2 && K0 != 16) return;   // (the two-piece block layout is that of K0 = 16 tiles)
  // The left-hand side is addressed with 32-bit byte offsets: a matrix of 2 GiB
  // or more (the library's entry point refuses it as well) does nothing here.
  if ((int64_t)M * K * Cfg::kElemBytes + 4096 > 0x7FFFFFFFll) return;
  MfmaArgs a;
  a.lhs = (const char*)lhs;
  a.rhs = (const char*)rhs;
  a.out = (char*)out;
  a.lhs_stride_bytes = (int64_t)K * Cfg::kElemBytes;            // row pitch of the matrix
  a.rhs_stride_bytes = (int64_t)K * 32 * Cfg::kElemBytes;       // one outer row of packed tiles
  a.out_stride_bytes = (int64_t)N * (int64_t)sizeof(out_t);
  a.M = (M + 31) / 32;
  a.N = (N + 31) / 32;
  a.panel_rows = 4;
  a.ksteps = K / Cfg::kMfmaK;
  a.tail_tiles = 0;
  a.tiles_m = (a.M * kPerTile + TM - 1) / TM;
  a.tiles_n = (a.N * kPerTile + TN - 1) / TN;
  a.accumulate = (flags & 0x100u) != 0;
  a.row_major_out = 1;
  a.out_rows = M;
  a.out_cols = N;
  a.lhs_row_major = 1;
  a.k_slices = 0; a.batch = 1; a.batch_by_xcd = 0;
  a.stream_out = 0;   // (row-major result)
  a.slice_ksteps = 0;
  a.slice_out_bytes = 0;
  a.k0_div = Cfg::kMfmaK / K0;
  a.gate_scale = a.up_scale = a.inv_out_scale = a.out_scale = 1.0f;
  if ((int)blockIdx.x >= a.tiles_m * a.tiles_n) return;
  mmt4d_mfma_body<Cfg, WM, WN, kRing, kSync, false, 2, 2>(a);
}

// Any other tile shape (the reference's pack and unpack take every tile size,
// runtime/src/iree/builtins/ukernel/pack.c:254-313, unpack.c:190-247): element
// by element over the same grid. A workgroup's block is `block_rows` rows of
// the (padded) matrix by 32 x 16 bytes of columns; thread (row, span) moves the
// 16 / ES elements of its span one by one to or from their places in the
// tiles, which are stored row by row, or column by column with kTransposed.
template <int ES, bool kPack, bool kTransposed>
__device__ __forceinline__ void hal_pack_elementwise(const void* mat, void* tiled, int size0, int size1,
                                                     int tile0, int tile1, uint32_t padding, uint32_t bx,
                                                     uint32_t by, int rows_per_block, int spans_per_block) {
  typedef typename Chunk<ES>::elem_t elem_t;
  constexpr int CE = 16 / ES;
  const uint32_t outer0 = ((uint32_t)size0 + tile0 - 1) / tile0, outer1 = ((uint32_t)size1 + tile1 - 1) / tile1;
  const int64_t rows = kPack ? (int64_t)outer0 * tile0 : size0;
  const int64_t cols = kPack ? (int64_t)outer1 * tile1 : size1;
  const int64_t tile_elems = (int64_t)tile0 * tile1;
  const elem_t* m_in = (const elem_t*)mat;
  elem_t* m_out = (elem_t*)mat;
  const elem_t* t_in = (const elem_t*)tiled;
  elem_t* t_out = (elem_t*)tiled;
  const int threads_per_row = 256 / rows_per_block;          // spans a row of threads covers per pass
  const int64_t r = (int64_t)by * rows_per_block + threadIdx.x / threads_per_row;
  if (r >= rows) return;
  const uint32_t orow = (uint32_t)r / tile0, trow = (uint32_t)r - orow * tile0;
  for (int sp = threadIdx.x % threads_per_row; sp < spans_per_block; sp += threads_per_row) {
    const int64_t c0 = ((int64_t)bx * spans_per_block + sp) * CE;
    for (int e = 0; e < CE; ++e) {
      const int64_t c = c0 + e;
      if (c >= cols) break;
      const uint32_t ocol = (uint32_t)c / tile1, tcol = (uint32_t)c - ocol * tile1;
      const int64_t at = ((int64_t)orow * outer1 + ocol) * tile_elems +
                         (kTransposed ? (int64_t)tcol * tile0 + trow : (int64_t)trow * tile1 + tcol);
      if (kPack) t_out[at] = (r < size0 && c < size1) ? m_in[r * size1 + c] : (elem_t)padding;
      else m_out[r * size1 + c] = t_in[at];
    }
  }
}

template <int ES, bool kPack>
__device__ __forceinline__ void hal_pack(const void* mat, void* tiled, int size0, int size1,
                                         int tile0, int tile1, uint32_t padding) {
  constexpr int CE = 16 / ES;
  if (size0 < 1 || size1 < 1 || tile0 < 1 || tile1 < 1) return;
  // Power-of-two tiles whose rows are whole 16-byte chunks: the streaming
  // kernel (the geometry below is shifts). Any other tile: element by element
  // over the same grid (blocks of 16 rows x 32 spans of 16 bytes).
  const int chunks = tile1 / CE;
  if ((tile0 & (tile0 - 1)) || tile1 % CE || (chunks & (chunks - 1))) {
    const int64_t outer0 = ((int64_t)size0 + tile0 - 1) / tile0, outer1 = ((int64_t)size1 + tile1 - 1) / tile1;
    const int64_t cols = kPack ? outer1 * tile1 : (int64_t)size1, rows = kPack ? outer0 * tile0 : (int64_t)size0;
    const uint32_t blocks_x = (uint32_t)(((cols * ES + 15) / 16 + 31) / 32), blocks_y = (uint32_t)((rows + 15) / 16);
    if (blockIdx.x >= blocks_x * blocks_y) return;
    hal_pack_elementwise<ES, kPack, false>(mat, tiled, size0, size1, tile0, tile1, padding, blockIdx.x % blocks_x,
                                           blockIdx.x / blocks_x, 16, 32);
    return;
  }
  Pow2Args a;
  a.log2_tile_rows = __builtin_ctz((unsigned)tile0);
  const int cpr = tile1 / CE;
  a.log2_cpr = __builtin_ctz((unsigned)cpr);
  const int64_t outer0 = ((int64_t)size0 + tile0 - 1) >> a.log2_tile_rows;
  const int64_t outer1 = ((int64_t)size1 + tile1 - 1) / tile1;
  a.mat = (const char*)mat;
  a.tiled = (char*)tiled;
  a.m_size0 = size0;
  a.m_size1 = size1;
  a.m_pitch_bytes = (int64_t)size1 * ES;
  a.t_stride_col_bytes = (int64_t)tile0 * tile1 * ES;
  a.t_stride_row_bytes = outer1 * a.t_stride_col_bytes;
  a.padded_rows = outer0 << a.log2_tile_rows;
  a.chunks_per_row = (uint32_t)(((int64_t)size1 + CE - 1) / CE);
  a.padded_chunks_per_row = (uint32_t)(outer1 * cpr);
  const int64_t cols = kPack ? a.padded_chunks_per_row : a.chunks_per_row;
  const int64_t rows = kPack ? a.padded_rows : (int64_t)size0;
  a.blocks_x = (uint32_t)((cols + 4 * kBlockChunks - 1) / (4 * kBlockChunks));
  a.blocks_y = (uint32_t)((rows + kBlockRows * kStreamUnroll - 1) / (kBlockRows * kStreamUnroll));
  a.padding = padding;
  if (blockIdx.x >= a.blocks_x * a.blocks_y) return;
  // (blocks of 16 rows x 32 chunks per 256 threads, as the export's workgroup
  // count says: 2 x 2 waves of 2 blocks of 4 rows x 16 chunks; tiles whose rows
  // are one chunk: 4 waves side by side, each 2 blocks of 8 rows x 8 chunks, so
  // that a wave's piece of a tile is a whole cache line)
  if (cpr == 1 && tile0 >= 8) stream_pow2_body<ES, kPack, true, kPack, 8, 2, 4, 4>(a);
  else stream_pow2_body<ES, kPack, true, kPack, 4, 2, 2, 4>(a);
}

// Transposed inner tiles: tile0 rows x tile1 columns of the matrix, stored
// column by column.
template <int ES, bool kPack>
__device__ __forceinline__ void hal_pack_transpose(const void* mat, void* tiled, int size0, int size1,
                                                   int tile0, int tile1, uint32_t padding) {
  constexpr int CE = 16 / ES;
  if (size0 < 1 || size1 < 1 || tile0 < 1 || tile1 < 1) return;
  // Power-of-two tiles of at least 16 bytes of rows (a stored column is then
  // whole 16-byte chunks and the divisions below are a multiplication by 2^31
  // and a shift): the chunk kernels. Any other tile: element by element over
  // the same grid, blocks of 64 columns x 16 groups of CE rows, a tile having
  // ceil(tile0 / CE) groups.
  if ((tile0 & (tile0 - 1)) || (tile1 & (tile1 - 1)) || tile0 < CE) {
    const int64_t outer0 = ((int64_t)size0 + tile0 - 1) / tile0, outer1 = ((int64_t)size1 + tile1 - 1) / tile1;
    const int64_t cols = kPack ? outer1 * tile1 : (int64_t)size1;
    const int64_t rows = kPack ? outer0 * tile0 : (int64_t)size0;
    // (rows rather than groups: 16 groups of CE rows are 16 CE rows of the padded matrix)
    const uint32_t blocks_x = (uint32_t)((cols + 63) / 64), blocks_y = (uint32_t)((rows + 16 * CE - 1) / (16 * CE));
    if (blockIdx.x >= blocks_x * blocks_y) return;
    // 64 columns = 64 / CE spans of CE elements; 16 CE rows per block
    hal_pack_elementwise<ES, kPack, true>(mat, tiled, size0, size1, tile0, tile1, padding, blockIdx.x % blocks_x,
                                          blockIdx.x / blocks_x, 16 * CE, 64 / CE);
    return;
  }
  auto by_pow2 = [](int d) {
    FastDiv f;
    f.d = (uint32_t)d;
    f.mul = 1u << 31;
    f.shift = 31 + __builtin_ctz((unsigned)d);
    return f;
  };
  TransArgs a;
  a.mat = (const char*)mat;
  a.tiled = (char*)tiled;
  a.m_size0 = size0;
  a.m_size1 = size1;
  a.m_pitch_bytes = (int64_t)size1 * ES;
  a.tile_rows = tile0;
  a.tile_cols = tile1;
  a.groups_per_tile = tile0 / CE;
  const int64_t outer_rows = ((int64_t)size0 + tile0 - 1) / tile0, outer_cols = ((int64_t)size1 + tile1 - 1) / tile1;
  a.row_groups = outer_rows * a.groups_per_tile;
  a.padded_cols = outer_cols * tile1;
  a.t_stride_ocol_bytes = (int64_t)tile0 * tile1 * ES;
  a.t_stride_orow_bytes = outer_cols * a.t_stride_ocol_bytes;
  a.by_tile_cols = by_pow2(tile1);
  a.by_groups = by_pow2(a.groups_per_tile);
  a.padding = padding;
  const int64_t cols = kPack ? a.padded_cols : (int64_t)size1;
  a.blocks_x = (uint32_t)((cols + 63) / 64);
  a.blocks_y = (uint32_t)((a.row_groups + 4 * kTransUnroll - 1) / (4 * kTransUnroll));
  if (blockIdx.x >= a.blocks_x * a.blocks_y) return;
  if (kPack) pack_transpose_body<ES>(a);
  else unpack_transpose_body<ES>(a);
}

// The decode configuration of the int4 dequantising matmul: K = 4096, groups
// of 128, packed uint4 zero points, tiled weights.
template <int MH>
__device__ __forceinline__ void hal_dequant_matmul_i4(const void* x, const void* w, const void* scale,
                                                      const void* zp, void* out, int M, int N) {
  constexpr int K = 4096;
  if (M < 1 || M > 16 * MH || N < 32 || N % 32 || (int64_t)N * (K / 2) + K * 16 >= (1ll << 32)) return;
  i4::I4Args a;
  a.x = (const uint16_t*)x;
  a.w = (const uint8_t*)w;
  a.scale = (const uint16_t*)scale;
  a.zp = zp;
  a.out = (uint16_t*)out;
  a.M = M; a.N = N; a.K = K; a.G = K / 128;
  a.log2_gs = 7;
  a.zp_u4 = 1;
  a.tiled = 1;
  a.n_tiles = N / 32;
  a.m_base = 0;
  a.stage_rows = i4::stage_rows_for(M);
  a.span_stride = 2048;
  a.col_stride = 64;
  a.w_bytes = (uint32_t)((int64_t)N * (K / 2));
  a.partial = nullptr;
  if ((int)blockIdx.x >= a.n_tiles || blockIdx.y != 0) return;
  i4::dequant_matmul_i4_body<8, MH, true, 7>(a);
}

}  // namespace

#define MI355X_DEQUANT_I4_EXPORT(NAME, MH)                                                         \
  extern "C" __global__ __launch_bounds__(512) void mi355x_dequant_matmul_i4_k4096_g128_##NAME(    \
      const void* __restrict__ x, const void* __restrict__ w, const void* __restrict__ scale,      \
      const void* __restrict__ zp, void* __restrict__ out, int M, int N) {                         \
    hal_dequant_matmul_i4<MH>(x, w, scale, zp, out, M, N);                                        \
  }
MI355X_DEQUANT_I4_EXPORT(r16, 1)
MI355X_DEQUANT_I4_EXPORT(r32, 2)

#define MI355X_PACK_EXPORTS(BITS, ES)                                                              \
  extern "C" __global__ __launch_bounds__(256) void mi355x_pack_##BITS##bit(                      \
      const void* __restrict__ in, void* __restrict__ out, int size0, int size1, int tile0,       \
      int tile1, unsigned padding) {                                                               \
    hal_pack<ES, true>(in, out, size0, size1, tile0, tile1, padding);                             \
  }
#define MI355X_UNPACK_EXPORTS(BITS, ES)                                                            \
  extern "C" __global__ __launch_bounds__(256) void mi355x_unpack_##BITS##bit(                    \
      const void* __restrict__ in, void* __restrict__ out, int size0, int size1, int tile0,       \
      int tile1) {                                                                                 \
    hal_pack<ES, false>(out, const_cast<void*>(in), size0, size1, tile0, tile1, 0);               \
  }
#define MI355X_PACK_TRANSPOSE_EXPORTS(BITS, ES)                                                    \
  extern "C" __global__ __launch_bounds__(256) void mi355x_pack_transpose_##BITS##bit(            \
      const void* __restrict__ in, void* __restrict__ out, int size0, int size1, int tile0,       \
      int tile1, unsigned padding) {                                                               \
    hal_pack_transpose<ES, true>(in, out, size0, size1, tile0, tile1, padding);                   \
  }
#define MI355X_UNPACK_TRANSPOSE_EXPORTS(BITS, ES)                                                  \
  extern "C" __global__ __launch_bounds__(256) void mi355x_unpack_transpose_##BITS##bit(          \
      const void* __restrict__ in, void* __restrict__ out, int size0, int size1, int tile0,       \
      int tile1) {                                                                                 \
    hal_pack_transpose<ES, false>(out, const_cast<void*>(in), size0, size1, tile0, tile1, 0);     \
  }
MI355X_PACK_EXPORTS(8, 1)
MI355X_PACK_EXPORTS(16, 2)
MI355X_PACK_EXPORTS(32, 4)
MI355X_UNPACK_EXPORTS(16, 2)
MI355X_UNPACK_EXPORTS(32, 4)
MI355X_PACK_TRANSPOSE_EXPORTS(8, 1)
MI355X_PACK_TRANSPOSE_EXPORTS(16, 2)
MI355X_PACK_TRANSPOSE_EXPORTS(32, 4)
MI355X_UNPACK_TRANSPOSE_EXPORTS(16, 2)
MI355X_UNPACK_TRANSPOSE_EXPORTS(32, 4)

#define MI355X_MATMUL_EXPORT(NAME, CFG, WM, WN, RING, SYNC, OCC, LDS)                              \
  static_assert(uk::mmt4d_mfma_lds_bytes<uk::CFG, WM, WN, RING>() == LDS, "LDS size of the table"); \
  extern "C" __global__ __launch_bounds__(256, OCC) void mi355x_matmul_packed_rhs_##NAME(          \
      const void* __restrict__ lhs, const void* __restrict__ rhs, void* __restrict__ out, int M,   \
      int N, int K, int K0, unsigned flags) {                                                      \
    hal_matmul_packed_rhs<uk::CFG, WM, WN, RING, SYNC>(lhs, rhs, out, M, N, K, K0, flags);        \
  }
// name            config    blocks/wave ring sync occ  LDS bytes
MI355X_MATMUL_EXPORT(f16f16f32_t4x8, F16Cfg16, 4, 8, 3, 1, 2, 73728)
MI355X_MATMUL_EXPORT(f16f16f32_t8x8, F16Cfg16, 8, 8, 5, 1, 1, 163840)
MI355X_MATMUL_EXPORT(bf16bf16f32_t4x8, BF16Cfg16, 4, 8, 3, 1, 2, 73728)
MI355X_MATMUL_EXPORT(bf16bf16f32_t8x8, BF16Cfg16, 8, 8, 5, 1, 1, 163840)
MI355X_MATMUL_EXPORT(s8s8s32_t4x8, S8Cfg, 2, 4, 6, 2, 2, 73728)
MI355X_MATMUL_EXPORT(s8s8s32_t8x8, S8Cfg, 4, 4, 8, 2, 1, 131072)
// (K0 = 16 and K a multiple of 64: the 16-row instruction, whose K-step is 64
// bytes of a row, so that a lane quad loads 64 contiguous bytes of a row of
// the left-hand side)
MI355X_MATMUL_EXPORT(s8s8s32_k64_t4x8, S8Cfg16, 4, 8, 3, 1, 2, 73728)
MI355X_MATMUL_EXPORT(s8s8s32_k64_t8x8, S8Cfg16, 8, 8, 5, 1, 1, 163840)
MI355X_MATMUL_EXPORT(f8e4m3f8e4m3f32_t4x8, F8Cfg, 2, 4, 3, 1, 2, 73728)
MI355X_MATMUL_EXPORT(f8e4m3f8e4m3f32_t8x8, F8Cfg, 4, 4, 5, 1, 1, 163840)
MI355X_MATMUL_EXPORT(f32f32f32_t4x8, F32Cfg, 2, 4, 6, 2, 2, 73728)
MI355X_MATMUL_EXPORT(f32f32f32_t8x8, F32Cfg, 4, 4, 8, 2, 1, 131072)

// One export per element-type tuple and macro tile, in the tiled and the
// row-major-result form.
#define MI355X_MMT4D_EXPORTS(NAME, CFG, WM, WN, RING, SYNC, OCC, LDS)                              \
  static_assert(uk::mmt4d_mfma_lds_bytes<uk::CFG, WM, WN, RING>() == LDS, "LDS size of the table"); \
  extern "C" __global__ __launch_bounds__(256, OCC) void mi355x_mmt4d_##NAME(                      \
      const void* __restrict__ lhs, const void* __restrict__ rhs, void* __restrict__ out, int M,   \
      int N, int K, int K0, unsigned flags) {                                                      \
    hal_mmt4d<uk::CFG, WM, WN, RING, SYNC, false>(lhs, rhs, out, M, N, K, K0, flags, 0, 0);       \
  }                                                                                                \
  extern "C" __global__ __launch_bounds__(256, OCC) void mi355x_mmt4d_unpack_##NAME(               \
      const void* __restrict__ lhs, const void* __restrict__ rhs, void* __restrict__ out, int M,   \
      int N, int K, int K0, unsigned flags, int out_rows, int out_cols) {                          \
    hal_mmt4d<uk::CFG, WM, WN, RING, SYNC, true>(lhs, rhs, out, M, N, K, K0, flags, out_rows,     \
                                                 out_cols);                                        \
  }

// name                      config      blocks/wave  ring sync occ    T   LDS bytes   K0 served
// f16f16f32_t8   (256x256)  F16Cfg16      8 x 8        5    1   1     8   163840      8, 16
// f16f16f32_t4   (128x128)  F16Cfg16      4 x 4        4    1   1     4    65536      8, 16
// bf16bf16f32_t8 / _t4      BF16Cfg16     as f16
// s8s8s32_t8     (256x256)  S8Cfg16       8 x 8        5    1   1     8   163840      16, 32
// s8s8s32_t4     (128x128)  S8Cfg16       4 x 4        4    1   1     4    65536      16, 32
// f8e4m3f8e4m3f32_t8        F8Cfg         4 x 4        5    1   1     8   163840      16
// f8e4m3f8e4m3f32_t4        F8Cfg         2 x 2        8    2   1     4   131072      16
// f32f32f32_t8              F32Cfg        4 x 4        8    2   1     8   131072      4, 8
// f32f32f32_t4              F32Cfg        2 x 2        8    2   1     4    65536      4, 8
MI355X_MMT4D_EXPORTS(f16f16f32_t8, F16Cfg16, 8, 8, 5, 1, 1, 163840)
MI355X_MMT4D_EXPORTS(f16f16f32_t4, F16Cfg16, 4, 4, 4, 1, 1, 65536)
MI355X_MMT4D_EXPORTS(bf16bf16f32_t8, BF16Cfg16, 8, 8, 5, 1, 1, 163840)
MI355X_MMT4D_EXPORTS(bf16bf16f32_t4, BF16Cfg16, 4, 4, 4, 1, 1, 65536)
MI355X_MMT4D_EXPORTS(s8s8s32_t8, S8Cfg16, 8, 8, 5, 1, 1, 163840)
MI355X_MMT4D_EXPORTS(s8s8s32_t4, S8Cfg16, 4, 4, 4, 1, 1, 65536)
MI355X_MMT4D_EXPORTS(f8e4m3f8e4m3f32_t8, F8Cfg, 4, 4, 5, 1, 1, 163840)
MI355X_MMT4D_EXPORTS(f8e4m3f8e4m3f32_t4, F8Cfg, 2, 2, 8, 2, 1, 131072)
MI355X_MMT4D_EXPORTS(f32f32f32_t8, F32Cfg, 4, 4, 8, 2, 1, 131072)
MI355X_MMT4D_EXPORTS(f32f32f32_t4, F32Cfg, 2, 2, 8, 2, 1, 65536)
