/*
 * iree_amd_uk.h - C ABI of the MI355X (gfx950) data-tiled matmul microkernels.
 *
 * This is the boundary a host runtime binds to: plain C, plain pointers and
 * sizes, no C++ or torch types. Every entry point mirrors one public entry point
 * of the reference microkernel library (runtime/src/iree/builtins/ukernel/ in
 * the IREE tree, cited per function as REF <file>:<line>) with the same argument
 * order and meaning. Two things differ, because the work runs on a GPU:
 *
 *   - buffer pointers are DEVICE pointers (hipMalloc'ed or otherwise visible to
 *     the current HIP device); the *_host variants at the end take host
 *     pointers and stage through device memory;
 *   - the trailing `cpu_data` argument of the reference is kept (and ignored) so
 *     that argument lists stay positionally identical, and one extra trailing
 *     `void* stream` (a hipStream_t, NULL = the null stream) is appended.
 *     Launches are asynchronous on that stream.
 *
 * All offsets, strides and sizes are in ELEMENTS, not bytes, as in the
 * reference. Every function that can fail returns an int: 0 on success, else
 * one of the IREE_AMD_UK_STATUS_* codes (numerically the low 5 bits of
 * iree_status_code_t, REF runtime/src/iree/hal/local/executable_plugin.h:221-259)
 * and the call has launched nothing. The reference validates only in debug
 * builds (REF mmt4d.c:12-48, pack.c:51-103, unpack.c:32-81); this library always
 * validates.
 */
#ifndef IREE_AMD_UK_H_
#define IREE_AMD_UK_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(_WIN32)
#define IREE_AMD_UK_EXPORT
#else
#define IREE_AMD_UK_EXPORT __attribute__((visibility("default")))
#endif

typedef int64_t iree_amd_uk_index_t; /* REF common.h:269-275 (iree_uk_index_t) */

/*===------------------------------------------------------------------------===
 * Status codes (subset of iree_status_code_t that this library returns).
 *===------------------------------------------------------------------------===*/
#define IREE_AMD_UK_STATUS_OK 0
#define IREE_AMD_UK_STATUS_INVALID_ARGUMENT 3
#define IREE_AMD_UK_STATUS_NOT_FOUND 5
#define IREE_AMD_UK_STATUS_FAILED_PRECONDITION 9
#define IREE_AMD_UK_STATUS_OUT_OF_RANGE 11
#define IREE_AMD_UK_STATUS_UNIMPLEMENTED 12
#define IREE_AMD_UK_STATUS_INTERNAL 13
#define IREE_AMD_UK_STATUS_UNAVAILABLE 14

/*===------------------------------------------------------------------------===
 * Flag words. Numerically identical to REF exported_bits.h:29-106, which the
 * reference declares "set in stone" (exported_bits.h:15-17).
 *===------------------------------------------------------------------------===*/

/* mmt4d: low byte = (lhs, rhs, out) element type tuple. REF exported_bits.h:29-41 */
#define IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK 0xFF
#define IREE_AMD_UK_FLAG_MMT4D_TYPE_NONE 0x00
#define IREE_AMD_UK_FLAG_MMT4D_TYPE_F32F32F32 0x01
#define IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32 0x02
#define IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F32 0x03
#define IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F16 0x04
#define IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16F32 0x05
#define IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16BF16 0x06
#define IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S16S32 0x07
#define IREE_AMD_UK_FLAG_MMT4D_TYPE_S16U4S32 0x08
#define IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S8S32 0x09
#define IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S4S32 0x0A
/* Extension: the reference enum ends at 0x0A (END = 0x0B, exported_bits.h:41).
 * fp8 e4m3fn x e4m3fn -> f32 takes the next free value. Operand decoding follows
 * OCP/IEEE e4m3fn (subnormals kept), which is what the gfx950 fp8 MFMAs do; the
 * reference's scalar helper flushes subnormals (REF base/internal/math.h:322). */
#define IREE_AMD_UK_FLAG_MMT4D_TYPE_F8E4M3F8E4M3F32 0x0B
#define IREE_AMD_UK_FLAG_MMT4D_TYPE_END 0x0C

/* mmt4d bit flags. REF exported_bits.h:44-46 */
#define IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE 0x100
#define IREE_AMD_UK_FLAG_MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION 0x200
#define IREE_AMD_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS 0x400

/* iree_amd_uk_mmt4d_info result bits. REF exported_bits.h:49 */
#define IREE_AMD_UK_FLAG_MMT4D_INFO_HAVE_ARCHITECTURE_SPECIFIC_TILE_FUNCTION 0x1

/* pack. REF exported_bits.h:56-66 */
#define IREE_AMD_UK_FLAG_PACK_TYPE_MASK 0xFF
#define IREE_AMD_UK_FLAG_PACK_TYPE_NONE 0x00
#define IREE_AMD_UK_FLAG_PACK_TYPE_F32F32 0x01
#define IREE_AMD_UK_FLAG_PACK_TYPE_I8I8 0x02 /* also used for 1-byte fp8 */
#define IREE_AMD_UK_FLAG_PACK_TYPE_I32I32 0x03
#define IREE_AMD_UK_FLAG_PACK_TYPE_F16F16 0x04
#define IREE_AMD_UK_FLAG_PACK_TYPE_BF16BF16 0x05
#define IREE_AMD_UK_FLAG_PACK_TRANSPOSE_INNER 0x100
#define IREE_AMD_UK_FLAG_PACK_TRANSPOSE_OUTER 0x200

/* unpack. REF exported_bits.h:73-83 (0x02 is reserved, no I8 unpack) */
#define IREE_AMD_UK_FLAG_UNPACK_TYPE_MASK 0xFF
#define IREE_AMD_UK_FLAG_UNPACK_TYPE_NONE 0x00
#define IREE_AMD_UK_FLAG_UNPACK_TYPE_F32F32 0x01
#define IREE_AMD_UK_FLAG_UNPACK_TYPE_I32I32 0x03
#define IREE_AMD_UK_FLAG_UNPACK_TYPE_F16F16 0x04
#define IREE_AMD_UK_FLAG_UNPACK_TYPE_BF16BF16 0x05
#define IREE_AMD_UK_FLAG_UNPACK_TRANSPOSE_INNER 0x100
#define IREE_AMD_UK_FLAG_UNPACK_TRANSPOSE_OUTER 0x200

/* query_tile_sizes. REF exported_bits.h:91-106 */
#define IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_MASK 0xFF
#define IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_NONE 0x00
#define IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_LHS 0x01
#define IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_RHS 0x02
#define IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_RESULT 0x03
#define IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MASK 0xFF00
#define IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERATION_NONE 0x0000
#define IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_F32F32F32 0x0100
#define IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_I8I8I32 0x0200
#define IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_F16F16F32 0x0300
#define IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_F16F16F16 0x0400
#define IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_BF16BF16F32 0x0500
#define IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_BF16BF16BF16 0x0600
/* Extension (no reference counterpart): fp8 e4m3fn matmul. */
#define IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERATION_MATMUL_F8E4M3F8E4M3F32 0x0B00

/*===------------------------------------------------------------------------===
 * mmt4d
 *
 *   out[i][j][i0][j0] (+)= sum_k sum_k0 lhs[i][k][i0][k0] * rhs[j][k][j0][k0]
 *
 * for i<M, j<N, k<K (M, N, K are OUTER tile counts), i0<M0, j0<N0, k0<K0. The
 * three inner dimensions of every operand are contiguous; `*_stride0` is the
 * distance in elements between consecutive outermost indices and need not be
 * tight. 4-bit RHS elements are packed two per byte, even k0 in the low nibble
 * (REF mmt4d_tile_generic.c:37-44,132-135). M==0, N==0 or (K==0 with
 * ACCUMULATE) return without touching `out`; K==0 without ACCUMULATE zero-fills
 * (REF mmt4d.c:105-113).
 *===------------------------------------------------------------------------===*/

/* Field order = REF mmt4d_internal.h:14-32 (iree_uk_mmt4d_params_t). */
typedef struct iree_amd_uk_mmt4d_params_t {
  const void* lhs_buffer;
  iree_amd_uk_index_t lhs_offset;
  iree_amd_uk_index_t lhs_stride0;
  const void* rhs_buffer;
  iree_amd_uk_index_t rhs_offset;
  iree_amd_uk_index_t rhs_stride0;
  void* out_buffer;
  iree_amd_uk_index_t out_offset;
  iree_amd_uk_index_t out_stride0;
  iree_amd_uk_index_t M;
  iree_amd_uk_index_t N;
  iree_amd_uk_index_t K;
  int32_t M0;
  int32_t N0;
  int32_t K0;
  uint32_t flags;
  const uint64_t* cpu_data; /* accepted, ignored */
} iree_amd_uk_mmt4d_params_t;

/* Replaces REF mmt4d.h:14-21 / mmt4d.c:151-177 (iree_uk_mmt4d).
 * A matrix-core call of few macro tiles and a long K splits K and keeps the
 * partial sums in a scratch buffer the library allocates once per stream
 * (16 to 512 MiB; kept until iree_amd_uk_release_scratch or, with more than 64
 * streams in use, until it is the least recently used one); every other call
 * allocates nothing. */
IREE_AMD_UK_EXPORT int iree_amd_uk_mmt4d(
    const void* lhs_buffer, iree_amd_uk_index_t lhs_offset,
    iree_amd_uk_index_t lhs_stride0, const void* rhs_buffer,
    iree_amd_uk_index_t rhs_offset, iree_amd_uk_index_t rhs_stride0,
    void* out_buffer, iree_amd_uk_index_t out_offset,
    iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t M,
    iree_amd_uk_index_t N, iree_amd_uk_index_t K, int32_t M0, int32_t N0,
    int32_t K0, uint32_t flags, const uint64_t* cpu_data, void* stream);

/* Replaces REF mmt4d_internal.h:34 / mmt4d.c:115-141 (iree_uk_mmt4d_p). */
IREE_AMD_UK_EXPORT int iree_amd_uk_mmt4d_p(
    const iree_amd_uk_mmt4d_params_t* params, void* stream);

/* iree_amd_uk_mmt4d_p for callers that cannot allocate. It has no counterpart
 * in the reference (whose ukernels never allocate, REF
 * runtime/src/iree/builtins/ukernel/README.md:17-26); it is for callers that
 * cannot call hipMalloc: code under HIP graph capture, tight serving loops,
 * harnesses that forbid it. Same parameters, kernels and results as
 * iree_amd_uk_mmt4d_p, but the partial sums of a K split go to a device array
 * of IREE_AMD_UK_NOALLOC_SCRATCH_BYTES that is part of the library's code
 * object (every GPU the library runs on holds its own copy until the process
 * ends) instead of the per-stream buffer iree_amd_uk_mmt4d_p allocates. The
 * call makes no hipMalloc, hipFree or other allocating call. A call whose K
 * split needs more than the array holds fails with status 8
 * (RESOURCE_EXHAUSTED) and has launched nothing; iree_amd_uk_last_error says how
 * many bytes it needed. Calls that do not split K (most) use no scratch at all;
 * the other users are S8S4S32 at the gfx950 tiles, whose right-hand side is
 * widened to int8 in the same array (one byte per weight), and the types with
 * a 16-bit left-hand side, whose int8 digit planes and their product go there:
 * each when it fits, otherwise the call runs the element-wise kernel, which
 * needs no scratch memory (slow, never an error).
 * All calls on one GPU share that GPU's array and nothing in it needs to start
 * at zero (every partial sum is written before it is read), but calls whose
 * kernels overlap on one GPU - two streams, two host threads - race on it:
 * keep them on one stream. The first call on a device looks up the array's
 * address (hipGetSymbolAddress); make one call before starting a graph capture. */
#define IREE_AMD_UK_NOALLOC_SCRATCH_BYTES (32u << 20)
IREE_AMD_UK_EXPORT int iree_amd_uk_mmt4d_noalloc_p(
    const iree_amd_uk_mmt4d_params_t* params, void* stream);

/* linalg.batch_mmt4d: `batch` mmt4d problems of the shape `params` gives, entry
 * b on operands lying b * {lhs,rhs,out}_batch_stride elements after those of
 * entry 0 (offsets added to params->*_offset). Replaces the loop the reference
 * generates around its mmt4d ukernel: it tiles the batch dimension to 1 and
 * rank-reduces each entry to mmt4d (REF compiler/src/iree/compiler/Codegen/
 * Common/CPU/CPUPrepareUkernels.cpp:23-43 tileBatchDimsForBatchMmt4dOp,
 * :165-245 ConvertBatchMmt4DtoMmt4DPattern), so every entry has exactly the
 * result of iree_amd_uk_mmt4d_p on it. Matrix-core tiles (M0 = 32, and the
 * narrow ones, M = 1 and M0 < 32, whose K one launch row holds) whose batch
 * strides are whole 16 bytes run as ONE launch (batch entries are planes of
 * the grid; K is not split in it, so it allocates nothing); everything else
 * runs as iree_amd_uk_mmt4d_p entry by entry. Entries must not overlap in `out`.
 * batch == 0 does nothing. */
IREE_AMD_UK_EXPORT int iree_amd_uk_batch_mmt4d(
    const iree_amd_uk_mmt4d_params_t* params, iree_amd_uk_index_t batch,
    iree_amd_uk_index_t lhs_batch_stride, iree_amd_uk_index_t rhs_batch_stride,
    iree_amd_uk_index_t out_batch_stride, void* stream);

/* Replaces REF mmt4d.h:23-25 / mmt4d.c:179-185 (iree_uk_mmt4d_info): bit 0 set
 * when a gfx950 MFMA kernel (not the generic one) serves this type and tile. */
IREE_AMD_UK_EXPORT uint32_t iree_amd_uk_mmt4d_info(int32_t M0, int32_t N0,
                                                   int32_t K0, uint32_t flags,
                                                   const uint64_t* cpu_data);

/*===------------------------------------------------------------------------===
 * pack: row-major (strided) 2-D source -> 4-D tiled destination with padding.
 *
 * With (O0,O1,T0,T1) = out_size0..3 and destination strides
 * (out_stride0, T0*T1, T1, 1); TRANSPOSE_OUTER swaps (O0,O1) and their strides,
 * TRANSPOSE_INNER swaps (T0,T1) and their strides; then for every
 * a<O0,b<O1,c<T0,d<T1 the element (a,b,c,d) receives in[a*T0+c][b*T1+d] when that
 * is inside in_size0 x in_size1 and the low element-bits of `padding_value`
 * otherwise (REF tools/pack_test.c:13-71, pack.h:16-25). out_stride1 must equal
 * out_size2*out_size3 (REF pack.c:72). Any out_size == 0 writes nothing
 * (REF pack.c:106-109).
 *===------------------------------------------------------------------------===*/

/* Field order = REF pack_internal.h:12-30 (iree_uk_pack_params_t). */
typedef struct iree_amd_uk_pack_params_t {
  const void* in_buffer;
  iree_amd_uk_index_t in_offset;
  iree_amd_uk_index_t in_stride0;
  iree_amd_uk_index_t in_stride1;
  void* out_buffer;
  iree_amd_uk_index_t out_offset;
  iree_amd_uk_index_t out_stride0;
  iree_amd_uk_index_t out_stride1;
  iree_amd_uk_index_t in_size0;
  iree_amd_uk_index_t in_size1;
  iree_amd_uk_index_t out_size0;
  iree_amd_uk_index_t out_size1;
  iree_amd_uk_index_t out_size2;
  iree_amd_uk_index_t out_size3;
  uint64_t padding_value;
  uint32_t flags;
  const uint64_t* cpu_data; /* accepted, ignored */
} iree_amd_uk_pack_params_t;

/* Replaces REF pack.h:26-34 / pack.c:325-352 (iree_uk_pack). */
IREE_AMD_UK_EXPORT int iree_amd_uk_pack(
    const void* in_buffer, iree_amd_uk_index_t in_offset,
    iree_amd_uk_index_t in_stride0, iree_amd_uk_index_t in_stride1,
    void* out_buffer, iree_amd_uk_index_t out_offset,
    iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t out_stride1,
    iree_amd_uk_index_t in_size0, iree_amd_uk_index_t in_size1,
    iree_amd_uk_index_t out_size0, iree_amd_uk_index_t out_size1,
    iree_amd_uk_index_t out_size2, iree_amd_uk_index_t out_size3,
    uint64_t padding_value, uint32_t flags, const uint64_t* cpu_data,
    void* stream);

/* Replaces REF pack_internal.h:32 / pack.c:315-323 (iree_uk_pack_p). */
IREE_AMD_UK_EXPORT int iree_amd_uk_pack_p(
    const iree_amd_uk_pack_params_t* params, void* stream);

/*===------------------------------------------------------------------------===
 * unpack: inverse of pack without padding. Copies only elements inside
 * out_size0 x out_size1; every other destination element is left untouched
 * (REF tools/unpack_test.c:13-58). in_stride1 must equal in_size2*in_size3
 * (REF unpack.c:49). out_size0 == 0 or out_size1 == 0 writes nothing
 * (REF unpack.c:84-86).
 *===------------------------------------------------------------------------===*/

/* Field order = REF unpack_internal.h:12-29 (iree_uk_unpack_params_t). */
typedef struct iree_amd_uk_unpack_params_t {
  const void* in_buffer;
  iree_amd_uk_index_t in_offset;
  iree_amd_uk_index_t in_stride0;
  iree_amd_uk_index_t in_stride1;
  void* out_buffer;
  iree_amd_uk_index_t out_offset;
  iree_amd_uk_index_t out_stride0;
  iree_amd_uk_index_t out_stride1;
  iree_amd_uk_index_t in_size0;
  iree_amd_uk_index_t in_size1;
  iree_amd_uk_index_t in_size2;
  iree_amd_uk_index_t in_size3;
  iree_amd_uk_index_t out_size0;
  iree_amd_uk_index_t out_size1;
  uint32_t flags;
  const uint64_t* cpu_data; /* accepted, ignored */
} iree_amd_uk_unpack_params_t;

/* Replaces REF unpack.h:17-25 / unpack.c:259-285 (iree_uk_unpack). */
IREE_AMD_UK_EXPORT int iree_amd_uk_unpack(
    const void* in_buffer, iree_amd_uk_index_t in_offset,
    iree_amd_uk_index_t in_stride0, iree_amd_uk_index_t in_stride1,
    void* out_buffer, iree_amd_uk_index_t out_offset,
    iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t out_stride1,
    iree_amd_uk_index_t in_size0, iree_amd_uk_index_t in_size1,
    iree_amd_uk_index_t in_size2, iree_amd_uk_index_t in_size3,
    iree_amd_uk_index_t out_size0, iree_amd_uk_index_t out_size1,
    uint32_t flags, const uint64_t* cpu_data, void* stream);

/* Replaces REF unpack_internal.h:31 / unpack.c:249-257 (iree_uk_unpack_p). */
IREE_AMD_UK_EXPORT int iree_amd_uk_unpack_p(
    const iree_amd_uk_unpack_params_t* params, void* stream);

/*===------------------------------------------------------------------------===
 * The compile-time side of tile selection, as two host-only functions with the
 * structure of the reference's (a compiler that materialises encodings for
 * gfx950 would call these where the CPU one calls its own).
 *
 * enumerate_matmul_tiles: the tiles the gfx950 kernels serve for an operation
 * (an IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERATION_* value): the full
 * 32 x 32 x K0 tile first, then its truncations in M to 16, 8, 4, 2, 1
 * (REF CPUMaterializeEncodingPass.cpp:168-281 enumerateMatmulTile*: every
 * target lists the tile aimed at its instruction and "Truncation of the above"
 * entries). Writes at most `capacity` tiles, *out_count = how many there are.
 *
 * choose_matmul_tile: REF CPUMaterializeEncodingPass.cpp:284-377
 * chooseMatmulTile, rule for rule. narrow_m / narrow_n: the static size of a
 * narrow dimension, 0 when it is not narrow. A narrow N that is narrower than
 * M (or the only narrow one) is reduced to the narrow-M case and the chosen
 * tile's M and N are exchanged. Tiles beyond `upper_bound` (3 values M, N, K;
 * NULL = none) are skipped; of the rest, those with the least padding penalty
 * max(tile.M - PowerOf2Ceil(narrow_m), 0) are kept, and of those the first
 * with the largest M * N * K wins. NOT_FOUND when every tile was skipped.
 * iree_amd_uk_query_tile_sizes_2d below answers with exactly these choices.
 *===------------------------------------------------------------------------===*/
typedef struct iree_amd_uk_matmul_tile_t {
  int32_t M, N, K;
} iree_amd_uk_matmul_tile_t;

IREE_AMD_UK_EXPORT int iree_amd_uk_enumerate_matmul_tiles(
    uint32_t operation, iree_amd_uk_matmul_tile_t* tiles, int32_t capacity, int32_t* out_count);

IREE_AMD_UK_EXPORT int iree_amd_uk_choose_matmul_tile(
    const iree_amd_uk_matmul_tile_t* tiles, int32_t count, iree_amd_uk_index_t narrow_m,
    iree_amd_uk_index_t narrow_n, const iree_amd_uk_index_t* upper_bound,
    iree_amd_uk_matmul_tile_t* out_tile);

/*===------------------------------------------------------------------------===
 * query_tile_sizes_2d: (operation, operand role) -> (tile_size0, tile_size1).
 * LHS -> (M0,K0), RHS -> (N0,K0), RESULT -> (M0,N0) of the matmul tile chosen
 * for gfx950 (REF query_tile_sizes.c:43-63 for the role mapping).
 * `size0` / `size1` are the operand's own dimensions (INT64_MIN = dynamic): a
 * static M (LHS / RESULT size0) or N (RHS size0, RESULT size1) below 32 narrows
 * that tile dimension to the next power of two >= the size, as the reference's
 * compile-time chooser does for narrow matmuls
 * (REF compiler/src/iree/compiler/Codegen/Common/CPU/CPUMaterializeEncodingPass.cpp:284-377).
 * Like that chooser (its lines 296-303) the library narrows at most ONE of M0
 * and N0 per matmul, the one of the smaller static size, and a narrow N0 is
 * served as the narrow-M0 problem with the operands exchanged
 * (REF compiler/src/iree/compiler/Codegen/Common/EncodingUtils.cpp:23-92): the
 * RESULT role, which sees both sizes, applies the rule itself; a caller whose M
 * AND N are both static and below 32 passes the LHS / RHS query of the wider of
 * the two a dynamic size0. Every tile this function returns has a matrix-core
 * kernel (iree_amd_uk_mmt4d_info).
 *===------------------------------------------------------------------------===*/

/* REF query_tile_sizes.h:18-23 */
typedef struct iree_amd_uk_query_tile_sizes_2d_params_t {
  uint32_t flags;
  iree_amd_uk_index_t size0;
  iree_amd_uk_index_t size1;
  const uint64_t* cpu_data; /* accepted, ignored */
} iree_amd_uk_query_tile_sizes_2d_params_t;

/* REF query_tile_sizes.h:25-28 */
typedef struct iree_amd_uk_query_tile_sizes_2d_out_params_t {
  iree_amd_uk_index_t tile_size0;
  iree_amd_uk_index_t tile_size1;
} iree_amd_uk_query_tile_sizes_2d_out_params_t;

/* Replaces REF query_tile_sizes.h:29-31 / query_tile_sizes.c:65-75. Host-only,
 * touches no device. Returns INVALID_ARGUMENT for an unknown operation/role. */
IREE_AMD_UK_EXPORT int iree_amd_uk_query_tile_sizes_2d(
    const iree_amd_uk_query_tile_sizes_2d_params_t* params,
    iree_amd_uk_query_tile_sizes_2d_out_params_t* out_params);

/* The whole tile of one matmul from its three sizes at once (INT64_MIN =
 * dynamic): enumerate_matmul_tiles + choose_matmul_tile with narrow_m / narrow_n
 * set from the static sizes below the full tile. The three roles of
 * iree_amd_uk_query_tile_sizes_2d each see one operand, so LHS and RHS queries
 * of a matmul whose M AND N are both static and below 32 would narrow both
 * dimensions; a caller that knows all sizes asks here and gets the one
 * consistent answer (the narrower dimension narrowed, the other full:
 * REF CPUMaterializeEncodingPass.cpp:296-303). Host-only. */
IREE_AMD_UK_EXPORT int iree_amd_uk_query_matmul_tile_sizes(
    uint32_t operation, iree_amd_uk_index_t M, iree_amd_uk_index_t N, iree_amd_uk_index_t K,
    iree_amd_uk_matmul_tile_t* out_tile);

/*===------------------------------------------------------------------------===
 * Grouped int4-weight dequantising matmul (the dispatch that quantised LLM
 * inference lowers to; there is no reference ukernel for it, the semantics are
 * the fused dequantisation + matmul pattern of
 * REF compiler/src/iree/compiler/GlobalOptimization/FuseDequantizationMatmul.cpp:53-159
 * and GlobalOptimization/test/fuse_dequantization_matmul.mlir:127-158):
 *
 *   out[m][n] = sum_g sum_k  x[m][g*gs+k] * ((float)w[n][g][k] - zp[n][g]) * s[n][g]
 *
 * x: f16 [M][K] row-major. w: unsigned 4-bit [N][K], two per byte, even k in the
 * low nibble (REF tests/e2e/linalg/subbyte_to_fp.mlir, mmt4d_tile_generic.c:132-135).
 * scales: f16 [N][K/gs]. zero points: either f16 [N][K/gs] (the reference's
 * form: a floating tensor subtracted after uitofp) or packed uint4 [N][K/gs]
 * (two per byte, even group in the low nibble) when ..._ZP_U4 is set. f32
 * accumulation, result rounded to f16 once (RNE). out: f16 [M][N] row-major.
 * Requires K % group_size == 0, group_size % 32 == 0, 1 <= M. A K beyond
 * 4096 is multiplied in slices whose f32 sums go through the stream's scratch
 * buffer (see iree_amd_uk_mmt4d on that buffer).
 *===------------------------------------------------------------------------===*/
#define IREE_AMD_UK_FLAG_DEQUANT_MATMUL_ZP_F16 0x0
#define IREE_AMD_UK_FLAG_DEQUANT_MATMUL_ZP_U4 0x1
/* Weights are in the pre-tiled layout that iree_amd_uk_pack_i4_weights
 * produces: tiles of 32 columns (n) x 128 k, 2 KiB each, ordered
 * [N/32][K/128]; inside a tile column c owns bytes [64c, 64c+64), in which the
 * 16 dwords of the row-major span (8 nibbles each, even k in the low nibble)
 * are transposed as a 4 x 4 matrix: dword q of 16-byte chunk j holds
 * k = 32q + 8j .. 32q + 8j + 7. A 64-lane wave then reads 1 KiB of contiguous
 * memory per load and every lane's four dwords feed four consecutive MFMAs.
 * Needs N % 32 == 0 and K % 128 == 0. Without the flag the weights are
 * row-major [N][K/2]; groups smaller than 128 are fast only from tiled weights. */
#define IREE_AMD_UK_FLAG_DEQUANT_MATMUL_W_TILED 0x2
/* The reassociated form, opt-in as in the reference ("introduces precision
 * loss", REF compiler/src/iree/compiler/GlobalOptimization/FuseDequantizationMatmul.cpp:746-767;
 * rewrite :398-645): the activations are quantised per group to 16 bits
 * (scale_x = max |x| / 32767, q = fptosi(x / scale_x)), the products are
 * integer (i16 x u4 -> i32 per group: the reference's S16U4S32 mmt4d,
 * REF runtime/src/iree/builtins/ukernel/arch/x86_64/mmt4d_x86_64_avx512_vnni.c:210-294)
 * and out = sum_g float(acc) * scale_x * s - (zp * s) * sum_k x, all float steps
 * in f32, rounded to f16 once. The quantised activations live in the stream's
 * scratch buffer (see iree_amd_uk_mmt4d); where that cannot be leased (the
 * per-thread default stream, another thread's call holding it) the call takes
 * its own with hipMallocAsync / hipFreeAsync on `stream`, and returns
 * RESOURCE_EXHAUSTED only when the device has no memory left. On the matrix cores from tiled
 * weights with K = 2048 or 4096 and power-of-two groups of 128 to K / 8;
 * everything else runs an element-wise kernel. */
#define IREE_AMD_UK_FLAG_DEQUANT_MATMUL_REASSOCIATE 0x4

IREE_AMD_UK_EXPORT int iree_amd_uk_dequant_matmul_i4(
    const void* x_buffer, const void* w_buffer, const void* scale_buffer,
    const void* zp_buffer, void* out_buffer, iree_amd_uk_index_t M,
    iree_amd_uk_index_t N, iree_amd_uk_index_t K,
    iree_amd_uk_index_t group_size, uint32_t flags, void* stream);

/* The quantisation step of the reassociated form by itself (the first three
 * dispatches of the rewrite, REF FuseDequantizationMatmul.cpp:398-492):
 * x f16 [M][K] -> q i16 [M][K], scale_x f32 [M][K/gs] = max |x| / 32767 per
 * group, group_sum f32 [M][K/gs] (lane-strided partial sums combined by a
 * butterfly; the reference adds in k order). A group of zeros gives zeros. */
IREE_AMD_UK_EXPORT int iree_amd_uk_quantize_groups_i16(
    const void* x_f16, void* q_i16, void* scale_x_f32, void* group_sum_f32,
    iree_amd_uk_index_t M, iree_amd_uk_index_t K, iree_amd_uk_index_t group_size,
    void* stream);

/* Row-major [N][K/2] 4-bit weights -> the ..._W_TILED layout above (done once
 * per weight matrix, like the reference's pack of a constant right-hand side
 * at compile time, REF compiler/src/iree/compiler/GlobalOptimization/
 * MaterializeHomogeneousEncodings.cpp). N % 32 == 0, K % 128 == 0; src and dst
 * must not overlap. */
IREE_AMD_UK_EXPORT int iree_amd_uk_pack_i4_weights(
    const void* w_rowmajor, void* w_tiled, iree_amd_uk_index_t N,
    iree_amd_uk_index_t K, void* stream);

/*===------------------------------------------------------------------------===
 * Pieces of the fp8 Llama-style MLP block (no reference ukernel; the pattern is
 * REF compiler/src/iree/compiler/GlobalOptimization/FuseSiluHorizontalMatmul.cpp:32-82,113-140:
 * h = silu(x Wg^T) * (x Wu^T), y = h Wd^T, silu(g) = g / (1 + exp(-g))).
 *===------------------------------------------------------------------------===*/

/* out_fp8[i] = e4m3fn_rne(clamp(in_f16[i] * inv_scale, +-448)), n elements.
 * Conversion is OCP e4m3fn round-to-nearest-even with saturation (values above
 * 448 in magnitude clamp to +-448 instead of the reference helper's NaN,
 * REF base/internal/math.h:363-423); NaN stays NaN. */
IREE_AMD_UK_EXPORT int iree_amd_uk_quantize_f16_to_f8e4m3(
    const void* in_f16, void* out_fp8, iree_amd_uk_index_t n, float inv_scale,
    void* stream);

/* The same conversion and the pack of its result in one pass: f16 row-major
 * [rows][cols] (row pitch `ld` elements) -> e4m3 left-hand-side tiles
 * [ceil(rows/32)][cols/16][32][16] with outer pitch `out_stride0` bytes; rows
 * past `rows` are zero. Bit-identical to iree_amd_uk_quantize_f16_to_f8e4m3
 * followed by iree_amd_uk_pack (8-bit, tiles 32x16, padding 0). cols must be
 * whole tiles of 16. */
IREE_AMD_UK_EXPORT int iree_amd_uk_quantize_pack_f8e4m3(
    const void* in_f16, iree_amd_uk_index_t ld, void* out_tiles,
    iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t rows,
    iree_amd_uk_index_t cols, float inv_scale, void* stream);

/* out_fp8[m][n] = e4m3fn( silu(gate[m][n]*gate_scale) * (up[m][n]*up_scale)
 *                          * inv_out_scale ), gate/up f32 row-major [rows][cols]
 * with row pitch `ld` elements. */
IREE_AMD_UK_EXPORT int iree_amd_uk_silu_mul_quantize(
    const void* gate_f32, const void* up_f32, void* out_fp8,
    iree_amd_uk_index_t rows, iree_amd_uk_index_t cols, iree_amd_uk_index_t ld,
    float gate_scale, float up_scale, float inv_out_scale, void* stream);

/* The same on data-tiled buffers, fusing the unpack of the gate/up result and
 * the pack of the next left-hand side: `acc_tiled` is an mmt4d f32 result with
 * 32x32 tiles (outer row pitch acc_stride0 ELEMENTS) whose outer columns
 * [gate_tile0, gate_tile0+N1) hold gate and [up_tile0, up_tile0+N1) hold up;
 * `out_tiled` receives e4m3 left-hand-side tiles 32x16 (outer row pitch
 * out_stride0 elements), outer column 2j and 2j+1 from tile column j. M1 is the
 * number of outer rows. Buffers 16-byte aligned. */
IREE_AMD_UK_EXPORT int iree_amd_uk_silu_mul_quantize_tiled(
    const void* acc_tiled, iree_amd_uk_index_t acc_stride0,
    iree_amd_uk_index_t gate_tile0, iree_amd_uk_index_t up_tile0,
    void* out_tiled, iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t M1,
    iree_amd_uk_index_t N1, float gate_scale, float up_scale,
    float inv_out_scale, void* stream);

/* The gate/up matmul and the SiLU * up step in one kernel: an mmt4d (same
 * operands and meaning as iree_amd_uk_mmt4d, tiles M0 = N0 = 32, types
 * F16F16F32, BF16BF16F32 or F8E4M3F8E4M3F32 at the K0 of the tile-size query)
 * whose right-hand side holds gate and up tiles INTERLEAVED along its outer
 * dimension (outer row 2j = gate tile j, 2j+1 = up tile j; N counts both, so it
 * is even), and whose epilogue stores
 *   e4m3fn( silu(acc_gate * gate_scale) * (acc_up * up_scale) * inv_out_scale )
 * as left-hand-side tiles 32x16 of the next matmul instead of the f32
 * accumulators: out holds N/2 * 1024 bytes per outer row, out_offset and
 * out_stride0 are in bytes. No accumulate flag. Operands must be 16-byte
 * aligned (there is no element-wise fallback for this fused form:
 * IREE_AMD_UK_STATUS_UNIMPLEMENTED otherwise). The f32 accumulators never
 * reach memory, which saves writing and re-reading 8 bytes per output byte. */
IREE_AMD_UK_EXPORT int iree_amd_uk_mmt4d_silu_mul_f8e4m3(
    const void* lhs_buffer, iree_amd_uk_index_t lhs_offset,
    iree_amd_uk_index_t lhs_stride0, const void* rhs_buffer,
    iree_amd_uk_index_t rhs_offset, iree_amd_uk_index_t rhs_stride0,
    void* out_buffer, iree_amd_uk_index_t out_offset,
    iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t M,
    iree_amd_uk_index_t N, iree_amd_uk_index_t K, int32_t K0, uint32_t flags,
    float gate_scale, float up_scale, float inv_out_scale, void* stream);

/* mmt4d fused with the unpack that would follow it (no counterpart ukernel in
 * the reference; its dispatches are linalg.mmt4d followed by tensor.unpack,
 * REF compiler/src/iree/compiler/Codegen/Common/CPU/CPULowerToUKernels.cpp:339-480):
 * operands and meaning as iree_amd_uk_mmt4d with tiles M0 = N0 = 32, but the
 * result is written (and, with the ACCUMULATE flag, first read) as the row-major
 * out_size0 x out_size1 matrix that iree_amd_uk_unpack without transpose flags
 * would produce from the tiled result: out_stride0 is the element pitch between
 * matrix rows, out_offset in elements, (M-1)*32 < out_size0 <= M*32 and
 * (N-1)*32 < out_size1 <= N*32. Float results are multiplied by out_scale on
 * the store (the product of the per-tensor scales of an fp8 matmul; must be 1
 * for integer types and with ACCUMULATE). With out_scale = 1 bit-identical to
 * the two-call sequence; saves writing and re-reading the tiled accumulator. Only tile shapes and types with
 * a matrix-core kernel (see iree_amd_uk_mmt4d_info) and 16-byte aligned
 * operands: IREE_AMD_UK_STATUS_UNIMPLEMENTED otherwise. */
IREE_AMD_UK_EXPORT int iree_amd_uk_mmt4d_unpack(
    const void* lhs_buffer, iree_amd_uk_index_t lhs_offset,
    iree_amd_uk_index_t lhs_stride0, const void* rhs_buffer,
    iree_amd_uk_index_t rhs_offset, iree_amd_uk_index_t rhs_stride0,
    void* out_buffer, iree_amd_uk_index_t out_offset,
    iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t out_size0,
    iree_amd_uk_index_t out_size1, iree_amd_uk_index_t M,
    iree_amd_uk_index_t N, iree_amd_uk_index_t K, int32_t K0, uint32_t flags,
    float out_scale, void* stream);

/* `batch` problems of iree_amd_uk_mmt4d_unpack, entry b on operands lying
 * b * {lhs,rhs,out}_batch_stride elements after those of entry 0 (what a
 * linalg.batch_mmt4d followed by the unpack of every entry computes; the
 * reference runs them entry by entry, REF CPUPrepareUkernels.cpp:23-43,165-245).
 * One launch whose workgroup planes are the entries; K is not split in it.
 * Every entry must satisfy what the single call asks of its operands (16-byte
 * aligned: the operand batch strides are whole 16 bytes, or 0 for an operand
 * all entries share). Entries must not overlap in `out`; batch == 0 does
 * nothing. */
IREE_AMD_UK_EXPORT int iree_amd_uk_batch_mmt4d_unpack(
    const void* lhs_buffer, iree_amd_uk_index_t lhs_offset,
    iree_amd_uk_index_t lhs_stride0, const void* rhs_buffer,
    iree_amd_uk_index_t rhs_offset, iree_amd_uk_index_t rhs_stride0,
    void* out_buffer, iree_amd_uk_index_t out_offset,
    iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t out_size0,
    iree_amd_uk_index_t out_size1, iree_amd_uk_index_t M,
    iree_amd_uk_index_t N, iree_amd_uk_index_t K, int32_t K0, uint32_t flags,
    float out_scale, iree_amd_uk_index_t batch, iree_amd_uk_index_t lhs_batch_stride,
    iree_amd_uk_index_t rhs_batch_stride, iree_amd_uk_index_t out_batch_stride, void* stream);

/* A whole matmul with a pre-packed right-hand side in one kernel: what the
 * reference runs as pack(LHS) -> mmt4d -> unpack
 * (REF compiler/src/iree/compiler/Codegen/Common/CPU/CPULowerToUKernels.cpp:339-480)
 * when the right-hand side (the weights) was packed ahead of time.
 *   out[m][n] (+)= sum_k lhs[m][k] * rhs_packed[n / 32][k / K0][n % 32][k % K0]
 * lhs is the row-major M x K matrix (lhs_stride0 = element pitch between
 * rows), rhs the packed buffer of ceil(N / 32) outer rows of K / K0 tiles
 * 32 x K0 (rhs_stride0 = element pitch between outer rows; columns past N must
 * be padded, with any values), out the row-major M x N result (out_stride0 =
 * element pitch). Offsets in elements. M, N, K count ELEMENTS here. flags: an
 * IREE_AMD_UK_FLAG_MMT4D_TYPE_* with a matrix-core kernel, optionally
 * ACCUMULATE / SKIP_INTERMEDIATE_ROUNDINGS. out_scale as for
 * iree_amd_uk_mmt4d_unpack. Requirements (IREE_AMD_UK_STATUS_UNIMPLEMENTED
 * otherwise; use the three-call sequence then): K a multiple of the
 * matrix-core K extent (32 for f16/bf16 and i8, 8 for f32, 64 for fp8),
 * K0 as served by iree_amd_uk_mmt4d, 16-byte aligned lhs rows and rhs tiles.
 * Bit-identical to pack + mmt4d + unpack. Up to 24 rows (32 of 1-byte elements: a decode step)
 * with a K of up to 4096 elements of 2 bytes (8192 of 1 byte) run the kernel
 * for narrow left-hand side tiles on the rows themselves (float sums then
 * come in that kernel's order: the bits of mmt4d on M0 = M tiles). With N >= 16384 (and M >= 512) the
 * left-hand side is packed into the stream's scratch buffer first (see
 * iree_amd_uk_mmt4d on that buffer). */
IREE_AMD_UK_EXPORT int iree_amd_uk_matmul_packed_rhs(
    const void* lhs_buffer, iree_amd_uk_index_t lhs_offset,
    iree_amd_uk_index_t lhs_stride0, const void* rhs_buffer,
    iree_amd_uk_index_t rhs_offset, iree_amd_uk_index_t rhs_stride0,
    void* out_buffer, iree_amd_uk_index_t out_offset,
    iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t M,
    iree_amd_uk_index_t N, iree_amd_uk_index_t K, int32_t K0, uint32_t flags,
    float out_scale, void* stream);

/* `batch` problems of iree_amd_uk_matmul_packed_rhs (a batch matmul on
 * row-major left-hand sides, every entry with packed weights of its own, or
 * rhs_batch_stride = 0 for shared ones), strides in elements as above. One
 * launch (the left-hand sides are read in the kernel, whatever N is); the same
 * conditions on every entry as the single call. */
IREE_AMD_UK_EXPORT int iree_amd_uk_batch_matmul_packed_rhs(
    const void* lhs_buffer, iree_amd_uk_index_t lhs_offset,
    iree_amd_uk_index_t lhs_stride0, const void* rhs_buffer,
    iree_amd_uk_index_t rhs_offset, iree_amd_uk_index_t rhs_stride0,
    void* out_buffer, iree_amd_uk_index_t out_offset,
    iree_amd_uk_index_t out_stride0, iree_amd_uk_index_t M,
    iree_amd_uk_index_t N, iree_amd_uk_index_t K, int32_t K0, uint32_t flags,
    float out_scale, iree_amd_uk_index_t batch, iree_amd_uk_index_t lhs_batch_stride,
    iree_amd_uk_index_t rhs_batch_stride, iree_amd_uk_index_t out_batch_stride, void* stream);

/* buf[i] *= scale over n f32 elements, in place (applies the product of the
 * per-tensor scales to an fp8 matmul result). */
IREE_AMD_UK_EXPORT int iree_amd_uk_scale_f32(void* buf_f32, iree_amd_uk_index_t n,
                                             float scale, void* stream);

/* NOT part of the reference interface (no iree_uk_* counterpart, nothing a
 * runtime binds to): a measurement aid for bench.py. It runs the mmt4d
 * kernel's matrix-core instruction pattern (every accumulator block of a wave's
 * 128 x 128 tile once per K-step, with the instruction shape the kernel uses for
 * the type; one workgroup of 4 waves per compute unit) for `iters` K-steps on operand
 * fragments that are read ONCE from `operands` and then stay in registers, so
 * the launch does no memory traffic. Timing it gives the rate the matrix cores
 * sustain for operands with that bit content, which on this part depends on
 * the data (the pipe is power-limited). `type_flag` is an
 * IREE_AMD_UK_FLAG_MMT4D_TYPE_* value with a matrix-core kernel; `operands`
 * holds at least 64 KiB (4 waves x up to 16 fragments x 64 lanes x 16 bytes, or
 * 8 fragments of 32 bytes for fp8); `sink` is at least 1 KiB and is normally left untouched; `*out_ops_per_launch`
 * receives the multiply-add operation count (2 per MAC) of one launch. */
IREE_AMD_UK_EXPORT int iree_amd_uk_mfma_probe(uint32_t type_flag,
                                              const void* operands,
                                              iree_amd_uk_index_t iters,
                                              void* sink,
                                              int64_t* out_ops_per_launch,
                                              void* stream);

/* NOT part of the reference interface either: the yardstick for the pack /
 * unpack streams, a plain out-of-place copy of `bytes` (a multiple of 8 KiB,
 * buffers 16-byte aligned and not overlapping) with 16-byte accesses, as the
 * reference's benchmarks measure memcpy next to pack
 * (REF runtime/src/iree/builtins/ukernel/tools/memcpy_benchmark.c:24-52).
 * mode 0 = plain accesses, 1 = non-temporal ones; 2 and 3 = the loads of 0
 * and 1 without the stores (the yardstick for kernels that only stream a
 * weight matrix; `dst` then needs 4 writable bytes and stays untouched); + 4 =
 * the same four in single-wave workgroups of 1 KiB per step (the pack / unpack
 * kernels' unit of work) instead of 256 threads and 8 KiB;
 * blocks_per_cu = workgroups per compute unit (0 = one workgroup per 8 KiB). */
IREE_AMD_UK_EXPORT int iree_amd_uk_copy_probe(const void* src, void* dst,
                                              iree_amd_uk_index_t bytes, int32_t mode,
                                              int32_t blocks_per_cu, void* stream);

/*===------------------------------------------------------------------------===
 * Thin device ABI, so that a pure-C host (the HAL executable plugin) needs no
 * HIP headers. Mirrors the handful of driver calls the reference's own HIP HAL
 * driver resolves at run time
 * (REF runtime/src/iree/hal/drivers/hip/dynamic_symbol_tables.h).
 *===------------------------------------------------------------------------===*/
IREE_AMD_UK_EXPORT int iree_amd_uk_device_count(int* out_count);
IREE_AMD_UK_EXPORT int iree_amd_uk_device_set(int ordinal);
IREE_AMD_UK_EXPORT int iree_amd_uk_device_malloc(void** out_ptr, uint64_t bytes);
IREE_AMD_UK_EXPORT int iree_amd_uk_device_free(void* ptr);
IREE_AMD_UK_EXPORT int iree_amd_uk_memcpy_h2d(void* dst, const void* src,
                                              uint64_t bytes, void* stream);
IREE_AMD_UK_EXPORT int iree_amd_uk_memcpy_d2h(void* dst, const void* src,
                                              uint64_t bytes, void* stream);
IREE_AMD_UK_EXPORT int iree_amd_uk_stream_create(void** out_stream);
IREE_AMD_UK_EXPORT int iree_amd_uk_stream_destroy(void* stream);
IREE_AMD_UK_EXPORT int iree_amd_uk_stream_synchronize(void* stream);
/* Frees the scratch buffers the library has cached per stream (see
 * iree_amd_uk_mmt4d) that no call is using at the moment; they come back on
 * demand. What a plugin calls from its unload. Waits for the device. */
IREE_AMD_UK_EXPORT int iree_amd_uk_release_scratch(void);
/* Human-readable text of the calling thread's last non-OK status ("" if none). */
IREE_AMD_UK_EXPORT const char* iree_amd_uk_last_error(void);
/* Name of the kernel family that served the calling thread's last mmt4d or
 * dequant_matmul_i4 call: "mmt4d:mfma", "mmt4d:mfma-narrow",
 * "mmt4d:mfma-widened-s4", "mmt4d:mfma-s16-planes", "mmt4d:element-wise",
 * "dequant_i4:mfma", "dequant_i4:gemv", "dequant_i4:reassociated",
 * "dequant_i4:element-wise" ("" before the first call). A static string. No
 * counterpart in the reference, whose tile-function choice is visible through
 * iree_uk_mmt4d_info only. */
IREE_AMD_UK_EXPORT const char* iree_amd_uk_last_kernel_path(void);
/* Library version: (major << 16) | minor. */
IREE_AMD_UK_EXPORT uint32_t iree_amd_uk_version(void);

/*===------------------------------------------------------------------------===
 * Host-pointer variants: same parameter structs, but every buffer is a HOST
 * pointer (what IREE's local-task/local-sync HAL hands an import,
 * REF samples/custom_dispatch/cpu/plugin/README.md:90-97). Each call stages the
 * touched byte ranges to device memory, runs the device entry point above,
 * copies the destination range back and synchronises before returning.
 * Reentrant; safe to call concurrently from several threads
 * (REF samples/custom_dispatch/cpu/plugin/system_plugin.c:21-25).
 *
 * The *_pooled forms take a pool that keeps the staging resources between
 * calls: up to 8 slots per device, each one stream and three device buffers
 * that grow on demand. A call owns a slot for its duration (calls beyond the
 * slots wait for one), so concurrent calls share nothing. A pool is what a
 * plugin instance owns: created in its load (touches no device), destroyed in
 * its unload once no call is running; there is no global state
 * (REF runtime/src/iree/hal/local/executable_plugin.h:415-418). The forms
 * without a pool build one for the single call (stream and buffers created and
 * freed per call). None of them splits K, so none uses the scratch cache.
 *===------------------------------------------------------------------------===*/
typedef struct iree_amd_uk_host_pool_t iree_amd_uk_host_pool_t;
IREE_AMD_UK_EXPORT int iree_amd_uk_host_pool_create(iree_amd_uk_host_pool_t** out_pool);
IREE_AMD_UK_EXPORT void iree_amd_uk_host_pool_destroy(iree_amd_uk_host_pool_t* pool);
IREE_AMD_UK_EXPORT int iree_amd_uk_mmt4d_host_pooled(
    iree_amd_uk_host_pool_t* pool, const iree_amd_uk_mmt4d_params_t* params);
IREE_AMD_UK_EXPORT int iree_amd_uk_pack_host_pooled(
    iree_amd_uk_host_pool_t* pool, const iree_amd_uk_pack_params_t* params);
IREE_AMD_UK_EXPORT int iree_amd_uk_unpack_host_pooled(
    iree_amd_uk_host_pool_t* pool, const iree_amd_uk_unpack_params_t* params);
IREE_AMD_UK_EXPORT int iree_amd_uk_mmt4d_host(
    const iree_amd_uk_mmt4d_params_t* params);
IREE_AMD_UK_EXPORT int iree_amd_uk_pack_host(
    const iree_amd_uk_pack_params_t* params);
IREE_AMD_UK_EXPORT int iree_amd_uk_unpack_host(
    const iree_amd_uk_unpack_params_t* params);

#ifdef __cplusplus
} /* extern "C" */
#endif

#endif /* IREE_AMD_UK_H_ */
