/*
 * oracle.h - CPU restatement of the reference's data-tiled matmul path.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing under iree_amd/ links, loads or calls this;
 * only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg do, and
 * only as the checker. It takes the same parameter structs as the device
 * library (include/iree_amd_uk.h) but every pointer is a HOST pointer.
 *
 * Each function states which reference lines it follows (paths relative to the
 * IREE tree). How each is pinned (what a wrong sign / index / transposition
 * would trip over) is listed in oracle.c's header.
 */
#ifndef IREE_AMD_ORACLE_H_
#define IREE_AMD_ORACLE_H_

#include <stdint.h>

#include "iree_amd_uk.h"

#ifdef __cplusplus
extern "C" {
#endif

/* f16 decoding mode for the float tile functions. */
#define ORACLE_F16_IEEE 0            /* subnormals kept (x86 vcvtph2ps, MFMA) */
#define ORACLE_F16_FLUSH_SUBNORMAL 1 /* reference generic path, common.h:685 */

/* REF runtime/src/iree/builtins/ukernel/mmt4d.c:55-141 (outer loops, early
 * return) + mmt4d_tile_generic.c:11-376 (one tile function per type tuple).
 * `f16_mode` selects how 16-bit floats are decoded. Returns 0, or non-zero when
 * the parameters are invalid per mmt4d.c:12-48. */
int oracle_mmt4d(const iree_amd_uk_mmt4d_params_t* params, int f16_mode);

/* Same contraction accumulated in double for the float types (f32, f16, bf16,
 * fp8 inputs), written as f32/f16/bf16 per the output type with one final
 * rounding. Used as the tolerance reference for random (non-exact) inputs. */
int oracle_mmt4d_f64(const iree_amd_uk_mmt4d_params_t* params);

/* REF runtime/src/iree/builtins/ukernel/tools/pack_test.c:13-71 (the normative
 * closed form) with the early return of pack.c:106-109. */
int oracle_pack(const iree_amd_uk_pack_params_t* params);

/* REF runtime/src/iree/builtins/ukernel/tools/unpack_test.c:13-58 with the early
 * return of unpack.c:84-86. */
int oracle_unpack(const iree_amd_uk_unpack_params_t* params);

/* REF runtime/src/iree/builtins/ukernel/query_tile_sizes.c:43-63: maps a matmul
 * tile (M0,N0,K0) to the 2-D tile of the operand whose role is in `flags`. */
int oracle_query_role_tile(uint32_t flags, int M0, int N0, int K0,
                           int64_t* tile_size0, int64_t* tile_size1);

/* REF runtime/src/iree/builtins/ukernel/common.h:665-792. */
float oracle_f16_to_f32(uint16_t v, int f16_mode);
uint16_t oracle_f32_to_f16(float v);
float oracle_bf16_to_f32(uint16_t v);
uint16_t oracle_f32_to_bf16(float v);

/* REF runtime/src/iree/base/internal/math.h:296-336 (decode) and :342-423
 * (encode, RNE, overflow -> NaN, subnormal results flushed to zero).
 * `ieee` != 0 keeps subnormals on both sides (OCP e4m3fn; what gfx950 does) and
 * `saturate` != 0 clamps finite overflow to +-448 instead of NaN. */
float oracle_f8e4m3_to_f32(uint8_t v, int ieee);
uint8_t oracle_f32_to_f8e4m3(float v, int ieee, int saturate);

/* REF runtime/src/iree/builtins/ukernel/tools/e2e_matmul_benchmark.c:94-127:
 * row-major C[M][N] (+)= A[M][K] * B[K][N]; type = mmt4d type flag value. */
int oracle_matmul_rowmajor(const void* a, const void* b, void* c, int64_t M,
                           int64_t N, int64_t K, uint32_t flags);

/* REF tools/testing/e2e/iree-e2e-matmul-test.cc:28-149 (reference_matmul_*):
 * row-major C[M][N] = (acc ? acc : 0) + A[M][K] * B[K][N]; floats accumulate in
 * f32 in k order, f16 / bf16 results are rounded once at the end; `acc` may be
 * NULL and has the result's element type. type = mmt4d type flag value
 * (S8S8S32, F32F32F32, F16F16F32, F16F16F16, BF16BF16F32, BF16BF16BF16). */
int oracle_e2e_reference_matmul(const void* a, const void* b, const void* acc,
                                void* c, int64_t M, int64_t N, int64_t K,
                                uint32_t flags);

/* REF tools/testing/e2e/test_utils.c:260-267 with the constants of
 * test_utils.h:99-100, used as iree-e2e-matmul-test.cc:641-660 does: n values
 * state % (max - min + 1) + min of the stream seeded with `seed`. */
uint32_t oracle_e2e_pseudorandom_fill(uint32_t seed, int64_t n, int32_t min,
                                      int32_t max, int32_t* out);

/* REF compiler/src/iree/compiler/GlobalOptimization/FuseDequantizationMatmul.cpp:53-159
 * and GlobalOptimization/test/fuse_dequantization_matmul.mlir:127-158: grouped
 * int4 dequant + matmul, evaluated in double, rounded once to f16. zp_is_u4
 * selects packed uint4 zero points instead of f16. */
int oracle_dequant_matmul_i4(const uint16_t* x, const uint8_t* w,
                             const uint16_t* scale, const void* zp,
                             uint16_t* out, int64_t M, int64_t N, int64_t K,
                             int64_t group_size, int zp_is_u4);

/* The opt-in reassociated form (REF FuseDequantizationMatmul.cpp:398-645,
 * 749-767): activations quantised per group to i16 (scale = absmax / 32767,
 * fptosi(x / scale)), i16 x u4 -> i32 products summed per group, then
 * sum_g (float(acc) * scale_x * scale - zp * scale * group_sum), all float
 * steps in f32 in the reference's order. q: [M][K], scale_x / group_sum:
 * [M][K/gs]. int_core (may be NULL) receives the integer sums [M][N][K/gs]. */
int oracle_quantize_groups_i16(const uint16_t* x, int64_t M, int64_t K, int64_t gs,
                               int16_t* q, float* scale_x, float* group_sum);
int oracle_dequant_matmul_i4_reassoc(const uint16_t* x, const uint8_t* w,
                                     const uint16_t* scale, const void* zp,
                                     uint16_t* out, int64_t M, int64_t N, int64_t K,
                                     int64_t gs, int zp_is_u4, int32_t* int_core);

/* REF compiler/src/iree/compiler/GlobalOptimization/FuseSiluHorizontalMatmul.cpp:32-82:
 * (g / (1 + exp(-g))) * u, in double. */
double oracle_silu_mul(double g, double u);

/* Multi-threaded (OpenMP over outer rows) wrappers used only for the timed CPU
 * baseline when the reference library itself is unavailable. */
int oracle_mmt4d_mt(const iree_amd_uk_mmt4d_params_t* params, int f16_mode,
                    int threads);

#ifdef __cplusplus
}
#endif
#endif /* IREE_AMD_ORACLE_H_ */
