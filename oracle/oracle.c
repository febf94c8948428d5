/*
 * oracle.c - CPU restatement of the reference's data-tiled matmul path.
 *
 * TEST INFRASTRUCTURE ONLY: see oracle.h. Written from the semantics of the
 * reference (cited per function), not from its text: one element-indexed loop
 * nest per operation, so that it shares no tiling, temporary-buffer or
 * tile-function structure with either the reference or the GPU kernels.
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   oracle_mmt4d (all integer types)   - against the reference library itself
 *       (oracle/_ref, generic and AVX-512/VNNI tile functions) on the
 *       reference's own shape/tile matrix, operands drawn with numpy
 *       generators over the reference's value ranges; against a numpy int64
 *       einsum; tile-shape invariance of the row-major result.
 *   oracle_mmt4d (float types)         - same, bit-exact, with the reference's
 *       small-integer value distributions (every partial sum exact); the
 *       no-skip-rounding f16/bf16 variants against oracle/_ref bit-exactly on
 *       random inputs (they are order-sensitive).
 *   oracle_mmt4d fp8 (extension)       - parity unpinned by the reference (the
 *       reference has no fp8 mmt4d); pinned by the e4m3 known answers below
 *       plus a numpy f64 einsum over the decoded table.
 *   oracle_pack / oracle_unpack        - against oracle/_ref on the reference's
 *       test matrix (transposes x padding regimes x strides x offsets); numpy
 *       reshape/transpose closed form; unpack(pack(x)) == x; canaries.
 *   f16/bf16 conversions               - exhaustive 65536-value decode against
 *       numpy.float16 / bit-shift bf16, encode against numpy RNE.
 *   f8e4m3 conversions                 - the known answers of
 *       runtime/src/iree/base/internal/math_test.cc:420-525 (committed as data
 *       in tests/golden/conversion_kat.json) and the closed form over all 256 codes.
 *   oracle_dequant_matmul_i4           - closed form in numpy float64; nibble
 *       order against tests/e2e/linalg/subbyte_to_fp.mlir's vectors.
 *   oracle_quantize_groups_i16 / oracle_dequant_matmul_i4_reassoc - no
 *       reference implementation can be run (the pattern is compiler IR): the
 *       quantisation against numpy float32 arithmetic, the integer core against
 *       oracle/_ref's iree_uk_mmt4d S16U4S32 on the 1x32x8 tile and a numpy
 *       integer product, the epilogue against the closed form in float64, and
 *       the whole against oracle_dequant_matmul_i4 on inputs the 16-bit
 *       quantisation represents exactly.
 *   oracle_silu_mul                    - libm identity x*sigmoid(x)*u.
 *   oracle_e2e_reference_matmul        - exact int64 products in numpy on the
 *       test runner's small-integer operands (every f32 partial sum exact, so
 *       the order of the additions cannot matter), rounded once by numpy.
 *   oracle_e2e_pseudorandom_fill       - a big-integer restatement in Python
 *       and the stream's first values worked out by hand.
 */
#include "oracle.h"

#include <math.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>

/*---------------------------------------------------------------------------*
 * Scalar conversions
 *---------------------------------------------------------------------------*/

static float bits_to_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static uint32_t f32_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}

/* Widen a 16-bit float with `ebits` exponent bits to f32.
 * REF common.h:665-702: NaN -> quiet NaN with all mantissa bits, Inf kept,
 * subnormals -> signed zero (flush mode) or their exact value (IEEE mode). */
static float widen16(uint16_t v, int ebits, int flush) {
  const int mbits = 15 - ebits;
  const uint32_t sign = (uint32_t)(v >> 15) << 31;
  const uint32_t e = (v >> mbits) & ((1u << ebits) - 1);
  const uint32_t m = v & ((1u << mbits) - 1);
  const int bias = (1 << (ebits - 1)) - 1;
  if (e == (1u << ebits) - 1) {
    return bits_to_f32(sign | 0x7F800000u | (m ? 0x007FFFFFu : 0));
  }
  if (e == 0) {
    if (flush || m == 0) return bits_to_f32(sign);
    float mag = ldexpf((float)m, 1 - bias - mbits);
    return sign ? -mag : mag;
  }
  return bits_to_f32(sign | ((e - bias + 127) << 23) | (m << (23 - mbits)));
}

/* Narrow f32 to a 16-bit float, RNE. REF common.h:704-770. The reference
 * measures exponents from 2^(bits-1) rather than from the IEEE bias, on both
 * sides: x = f32_exponent_field - 128, result field = x + 2^(ebits-1). Its
 * range tests are x >= 2^(ebits-1) -> Inf and x < -2^(ebits-1) -> 0, which for
 * f16 leaves two quirks that are restated here on purpose: magnitudes in
 * (65536, 131072) come out with exponent field 31 and a non-zero mantissa
 * (a NaN pattern), and magnitudes in [2^-15, 2^-14) come out with exponent
 * field 0 and the mantissa of the normal number. f32 subnormals give zero,
 * NaN gives the all-ones-mantissa quiet NaN. */
static uint16_t narrow16(float f, int ebits) {
  const int mbits = 15 - ebits;
  const uint32_t u = f32_to_bits(f);
  const uint16_t sign = (uint16_t)((u >> 31) << 15);
  const uint32_t fe = (u >> 23) & 0xFF;
  uint32_t fm = u & 0x7FFFFF;
  const uint16_t emask = (uint16_t)(((1u << ebits) - 1) << mbits);
  const uint16_t mmask = (uint16_t)((1u << mbits) - 1);
  if (fe == 0xFF) return sign | emask | (fm ? mmask : 0);
  if (fe == 0) return sign;
  int x = (int)fe - 128;
  const int half = 1 << (ebits - 1);
  if (x >= half) return sign | emask;
  if (x < -half) return sign;
  const uint32_t even = 1u << (23 - mbits);
  const uint32_t odd = even >> 1;
  fm += (fm & even) ? odd : (odd - 1);
  if (fm > 0x7FFFFF) {
    fm = 0;
    ++x;
  }
  return sign | (uint16_t)((uint32_t)(x + half) << mbits) |
         (uint16_t)(fm >> (23 - mbits));
}

float oracle_f16_to_f32(uint16_t v, int f16_mode) {
  return widen16(v, 5, f16_mode == ORACLE_F16_FLUSH_SUBNORMAL);
}
uint16_t oracle_f32_to_f16(float v) { return narrow16(v, 5); }
float oracle_bf16_to_f32(uint16_t v) { return widen16(v, 8, 1); }
uint16_t oracle_f32_to_bf16(float v) { return narrow16(v, 8); }

/* IEEE-correct f32->f16 RNE including subnormal results; used where the GPU
 * rounds in hardware (int4 matmul output). */
static uint16_t f32_to_f16_ieee(float f) {
  const uint32_t u = f32_to_bits(f);
  const uint16_t sign = (uint16_t)((u >> 16) & 0x8000);
  const uint32_t a = u & 0x7FFFFFFF;
  if (a > 0x7F800000) return sign | 0x7E00;
  if (a >= 0x477FF000) return sign | 0x7C00; /* >= 65520 -> inf */
  if (a < 0x33000001) return sign;           /* <= 2^-25 -> 0 (tie to even) */
  int e = (int)(a >> 23) - 127;
  uint32_t m = (a & 0x7FFFFF) | 0x800000;
  int shift = (e < -14) ? (13 + (-14 - e)) : 13;
  uint32_t q = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1);
  uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (q & 1))) ++q;
  if (e < -14) return sign | (uint16_t)q;
  /* q has the implicit bit at position 10; adding carries into the exponent. */
  return sign | (uint16_t)(((uint32_t)(e + 15) << 10) + (q - 0x400));
}

static float f8e4m3_decode_one(uint8_t v, int ieee);
/* The matmul loops decode two operands per multiply-add: the 2 x 256 values
 * are tabulated when the library is loaded. */
static float f8e4m3_table[2][256];
__attribute__((constructor)) static void f8e4m3_table_init(void) {
  for (int ieee = 0; ieee < 2; ++ieee)
    for (int v = 0; v < 256; ++v) f8e4m3_table[ieee][v] = f8e4m3_decode_one((uint8_t)v, ieee);
}

float oracle_f8e4m3_to_f32(uint8_t v, int ieee) { return f8e4m3_table[ieee ? 1 : 0][v]; }

static float f8e4m3_decode_one(uint8_t v, int ieee) {
  const int s = v >> 7, e = (v >> 3) & 0xF, m = v & 7;
  float mag;
  if (e == 15 && m == 7) return bits_to_f32(((uint32_t)s << 31) | 0x7FFFFFFFu);
  if (e == 0) {
    mag = ieee ? ldexpf((float)m, -9) : 0.0f;
  } else {
    mag = ldexpf((float)(8 + m), e - 7 - 3);
  }
  return s ? -mag : mag;
}

uint8_t oracle_f32_to_f8e4m3(float f, int ieee, int saturate) {
  const uint32_t u = f32_to_bits(f);
  const uint8_t sign = (uint8_t)((u >> 31) << 7);
  const uint32_t a = u & 0x7FFFFFFF;
  if (a > 0x7F800000) return sign | 0x7F;               /* NaN */
  if (a == 0x7F800000) return sign | (saturate ? 0x7E : 0x7F);
  const float mag = fabsf(f);
  if (!ieee) {
    /* REF math.h:363-423: f32 subnormals -> 0; unbiased exponent > 8 -> NaN
     * (no infinities); exponent < -8 -> 0; otherwise round the mantissa to 3
     * bits (RNE, carry bumps the exponent) and emit field = exponent + 7. For
     * exponent -7 that field is 0 with the mantissa kept (a subnormal code,
     * which the reference's own decoder reads as zero). For exponent -8 the
     * reference shifts a negative int, which is undefined in C; this
     * restatement returns zero there and no test relies on that range. */
    if ((a >> 23) == 0) return sign;
    int ex = (int)(a >> 23) - 127;
    if (ex > 8) return sign | (saturate ? 0x7E : 0x7F);
    if (ex < -8) return sign;
    uint32_t fm = a & 0x7FFFFF;
    const uint32_t even = 1u << 20, odd = even >> 1;
    fm += (fm & even) ? odd : (odd - 1);
    if (fm > 0x7FFFFF) {
      fm = 0;
      ++ex;
    }
    if (ex > 8) return sign | (saturate ? 0x7E : 0x7F);
    if (ex < -7) return sign;
    uint32_t code = ((uint32_t)(ex + 7) << 3) | (fm >> 20);
    if (code == 0x7F && saturate) code = 0x7E;
    return sign | (uint8_t)code;
  }
  /* IEEE/OCP: round to nearest even on the e4m3 grid including subnormals. */
  if (mag >= 464.0f) {
    /* 464 is the midpoint between 448 and the (non-existent) 480: ties go to
     * the even mantissa, which is 480's code 0x7F = NaN. */
    if (mag == 464.0f) return sign | 0x7E; /* REF math_test.cc:458 says 0x7E */
    return sign | (saturate ? 0x7E : 0x7F);
  }
  int ex;
  (void)frexpf(mag, &ex); /* mag = fr * 2^ex, fr in [0.5,1) */
  int e = ex - 1;         /* unbiased exponent of leading bit */
  if (e < -6) e = -6;     /* subnormal grid spacing 2^-9 */
  const float ulp = ldexpf(1.0f, e - 3);
  float q = mag / ulp; /* exact: power-of-two scaling */
  float r = nearbyintf(q);
  float val = r * ulp;
  if (val == 0.0f) return sign;
  if (val > 448.0f) return sign | (saturate ? 0x7E : 0x7F);
  (void)frexpf(val, &ex);
  e = ex - 1;
  if (e < -6) {
    return sign | (uint8_t)lrintf(ldexpf(val, 9));
  }
  int m = (int)lrintf(ldexpf(val, 3 - e)) - 8;
  return sign | (uint8_t)(((e + 7) << 3) | m);
}

/*---------------------------------------------------------------------------*
 * mmt4d
 *---------------------------------------------------------------------------*/

typedef struct {
  int lhs_bits, rhs_bits, out_bytes;
  int is_float; /* accumulate in float */
} type_info_t;

static int mmt4d_type_info(uint32_t flags, type_info_t* ti) {
  switch (flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK) {
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F32F32F32:
      *ti = (type_info_t){32, 32, 4, 1};
      return 0;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32:
      *ti = (type_info_t){8, 8, 4, 0};
      return 0;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F32:
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16F32:
      *ti = (type_info_t){16, 16, 4, 1};
      return 0;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F16:
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16BF16:
      *ti = (type_info_t){16, 16, 2, 1};
      return 0;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S16S32:
      *ti = (type_info_t){16, 16, 4, 0};
      return 0;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S16U4S32:
      *ti = (type_info_t){16, 4, 4, 0};
      return 0;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S8S32:
      *ti = (type_info_t){16, 8, 4, 0};
      return 0;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S4S32:
      *ti = (type_info_t){8, 4, 4, 0};
      return 0;
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F8E4M3F8E4M3F32:
      *ti = (type_info_t){8, 8, 4, 1};
      return 0;
    default:
      return 1;
  }
}

/* REF mmt4d.c:12-48, enforced unconditionally. */
static int mmt4d_validate(const iree_amd_uk_mmt4d_params_t* p, type_info_t* ti) {
  const uint32_t known = IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK |
                         IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE |
                         IREE_AMD_UK_FLAG_MMT4D_ALLOW_GENERIC_FALLBACK_TILE_FUNCTION |
                         IREE_AMD_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS;
  if (p->flags & ~known) return 1;
  if (mmt4d_type_info(p->flags, ti)) return 1;
  if (p->M < 0 || p->N < 0 || p->K < 0) return 1;
  if (p->M > 0x7FFFFFFF || p->N > 0x7FFFFFFF || p->K > 0x7FFFFFFF) return 1;
  if (p->M0 < 0 || p->N0 < 0 || p->K0 < 0) return 1;
  if (p->M0 > 0x7FFF || p->N0 > 0x7FFF || p->K0 > 0x7FFF) return 1;
  if ((p->K0 * ti->lhs_bits) % 8 || (p->K0 * ti->rhs_bits) % 8) return 1;
  if ((p->lhs_stride0 * ti->lhs_bits) % 8 || (p->rhs_stride0 * ti->rhs_bits) % 8)
    return 1;
  if ((p->lhs_offset * ti->lhs_bits) % 8 || (p->rhs_offset * ti->rhs_bits) % 8)
    return 1;
  return 0;
}

/* Integer element fetch: `idx` is an element index from the buffer start. */
static int32_t load_int(const void* base, int64_t idx, uint32_t type, int rhs) {
  switch (type) {
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32:
      return ((const int8_t*)base)[idx];
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S16S32:
      return ((const int16_t*)base)[idx];
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S8S32:
      return rhs ? ((const int8_t*)base)[idx] : ((const int16_t*)base)[idx];
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S16U4S32: {
      if (!rhs) return ((const int16_t*)base)[idx];
      uint8_t b = ((const uint8_t*)base)[idx >> 1];
      return (idx & 1) ? (b >> 4) : (b & 0xF);
    }
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S4S32: {
      if (!rhs) return ((const int8_t*)base)[idx];
      uint8_t b = ((const uint8_t*)base)[idx >> 1];
      int32_t nib = (idx & 1) ? (b >> 4) : (b & 0xF);
      return (nib & 8) ? nib - 16 : nib;
    }
    default:
      return 0;
  }
}

static float load_flt(const void* base, int64_t idx, uint32_t type, int mode) {
  switch (type) {
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F32F32F32:
      return ((const float*)base)[idx];
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F32:
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F16:
      return oracle_f16_to_f32(((const uint16_t*)base)[idx], mode);
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16F32:
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16BF16:
      return oracle_bf16_to_f32(((const uint16_t*)base)[idx]);
    case IREE_AMD_UK_FLAG_MMT4D_TYPE_F8E4M3F8E4M3F32:
      return oracle_f8e4m3_to_f32(((const uint8_t*)base)[idx], 1);
    default:
      return 0.f;
  }
}

static void mmt4d_rows(const iree_amd_uk_mmt4d_params_t* p, const type_info_t* ti,
                       int f16_mode, int use_f64, int64_t i_begin,
                       int64_t i_end) {
  const uint32_t type = p->flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK;
  const int acc_flag = (p->flags & IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE) != 0;
  const int skipround =
      (p->flags & IREE_AMD_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS) != 0;
  const int out16_f = type == IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F16;
  const int out16_b = type == IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16BF16;
  const int64_t M0 = p->M0, N0 = p->N0, K0 = p->K0;
  for (int64_t i = i_begin; i < i_end; ++i) {
    for (int64_t j = 0; j < p->N; ++j) {
      for (int64_t i0 = 0; i0 < M0; ++i0) {
        for (int64_t j0 = 0; j0 < N0; ++j0) {
          const int64_t o =
              p->out_offset + i * p->out_stride0 + j * M0 * N0 + i0 * N0 + j0;
          const int64_t lbase = p->lhs_offset + i * p->lhs_stride0 + i0 * K0;
          const int64_t rbase = p->rhs_offset + j * p->rhs_stride0 + j0 * K0;
          if (!ti->is_float) {
            int32_t* out = (int32_t*)p->out_buffer;
            /* Unsigned wrap-around arithmetic: the reference's int32 sums wrap
             * on x86; doing it in uint32 keeps that behaviour defined. */
            uint32_t acc = acc_flag ? (uint32_t)out[o] : 0u;
            for (int64_t k = 0; k < p->K; ++k) {
              for (int64_t k0 = 0; k0 < K0; ++k0) {
                int32_t l = load_int(p->lhs_buffer, lbase + k * M0 * K0 + k0, type, 0);
                int32_t r = load_int(p->rhs_buffer, rbase + k * N0 * K0 + k0, type, 1);
                acc += (uint32_t)(l * r);
              }
            }
            out[o] = (int32_t)acc;
          } else if (use_f64) {
            double acc = 0.0;
            if (acc_flag) {
              if (out16_f)
                acc = oracle_f16_to_f32(((uint16_t*)p->out_buffer)[o], ORACLE_F16_IEEE);
              else if (out16_b)
                acc = oracle_bf16_to_f32(((uint16_t*)p->out_buffer)[o]);
              else
                acc = ((float*)p->out_buffer)[o];
            }
            for (int64_t k = 0; k < p->K; ++k) {
              for (int64_t k0 = 0; k0 < K0; ++k0) {
                double l = load_flt(p->lhs_buffer, lbase + k * M0 * K0 + k0, type, ORACLE_F16_IEEE);
                double r = load_flt(p->rhs_buffer, rbase + k * N0 * K0 + k0, type, ORACLE_F16_IEEE);
                acc += l * r;
              }
            }
            if (out16_f)
              ((uint16_t*)p->out_buffer)[o] = f32_to_f16_ieee((float)acc);
            else if (out16_b)
              ((uint16_t*)p->out_buffer)[o] = oracle_f32_to_bf16((float)acc);
            else
              ((float*)p->out_buffer)[o] = (float)acc;
          } else if ((out16_f || out16_b) && !skipround) {
            /* REF mmt4d_tile_generic.c:229-257,318-346: the accumulator lives
             * in the 16-bit type and is re-rounded after every multiply-add. */
            uint16_t* out = (uint16_t*)p->out_buffer;
            uint16_t acc = acc_flag ? out[o] : 0;
            for (int64_t k = 0; k < p->K; ++k) {
              for (int64_t k0 = 0; k0 < K0; ++k0) {
                float l = load_flt(p->lhs_buffer, lbase + k * M0 * K0 + k0, type, f16_mode);
                float r = load_flt(p->rhs_buffer, rbase + k * N0 * K0 + k0, type, f16_mode);
                float a = out16_f ? oracle_f16_to_f32(acc, f16_mode)
                                  : oracle_bf16_to_f32(acc);
                float prod = l * r;
                float sum = a + prod;
                acc = out16_f ? oracle_f32_to_f16(sum) : oracle_f32_to_bf16(sum);
              }
            }
            out[o] = acc;
          } else {
            /* f32 accumulation, k-major then k0, multiply then add
             * (REF mmt4d_tile_generic.c:172-225,259-286,289-316,348-376). */
            float acc = 0.f;
            if (acc_flag) {
              if (out16_f)
                acc = oracle_f16_to_f32(((uint16_t*)p->out_buffer)[o], f16_mode);
              else if (out16_b)
                acc = oracle_bf16_to_f32(((uint16_t*)p->out_buffer)[o]);
              else
                acc = ((float*)p->out_buffer)[o];
            }
            for (int64_t k = 0; k < p->K; ++k) {
              for (int64_t k0 = 0; k0 < K0; ++k0) {
                float l = load_flt(p->lhs_buffer, lbase + k * M0 * K0 + k0, type, f16_mode);
                float r = load_flt(p->rhs_buffer, rbase + k * N0 * K0 + k0, type, f16_mode);
                float prod = l * r;
                acc = acc + prod;
              }
            }
            if (out16_f)
              ((uint16_t*)p->out_buffer)[o] = oracle_f32_to_f16(acc);
            else if (out16_b)
              ((uint16_t*)p->out_buffer)[o] = oracle_f32_to_bf16(acc);
            else
              ((float*)p->out_buffer)[o] = acc;
          }
        }
      }
    }
  }
}

/* REF mmt4d.c:105-113 */
static int mmt4d_is_noop(const iree_amd_uk_mmt4d_params_t* p) {
  return p->M == 0 || p->N == 0 ||
         (p->K == 0 && (p->flags & IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE));
}

int oracle_mmt4d(const iree_amd_uk_mmt4d_params_t* p, int f16_mode) {
  type_info_t ti;
  if (mmt4d_validate(p, &ti)) return IREE_AMD_UK_STATUS_INVALID_ARGUMENT;
  if (mmt4d_is_noop(p)) return 0;
  mmt4d_rows(p, &ti, f16_mode, 0, 0, p->M);
  return 0;
}

int oracle_mmt4d_f64(const iree_amd_uk_mmt4d_params_t* p) {
  type_info_t ti;
  if (mmt4d_validate(p, &ti)) return IREE_AMD_UK_STATUS_INVALID_ARGUMENT;
  if (mmt4d_is_noop(p)) return 0;
#pragma omp parallel for schedule(dynamic, 1)
  for (int64_t i = 0; i < p->M; ++i) mmt4d_rows(p, &ti, ORACLE_F16_IEEE, 1, i, i + 1);
  return 0;
}

int oracle_mmt4d_mt(const iree_amd_uk_mmt4d_params_t* p, int f16_mode,
                    int threads) {
  type_info_t ti;
  if (mmt4d_validate(p, &ti)) return IREE_AMD_UK_STATUS_INVALID_ARGUMENT;
  if (mmt4d_is_noop(p)) return 0;
  if (threads < 1) threads = 1;
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
  for (int64_t i = 0; i < p->M; ++i) mmt4d_rows(p, &ti, f16_mode, 0, i, i + 1);
  return 0;
}

/*---------------------------------------------------------------------------*
 * pack / unpack
 *---------------------------------------------------------------------------*/

static int pack_elem_size(uint32_t type) {
  switch (type) {
    case IREE_AMD_UK_FLAG_PACK_TYPE_F32F32:
    case IREE_AMD_UK_FLAG_PACK_TYPE_I32I32:
      return 4;
    case IREE_AMD_UK_FLAG_PACK_TYPE_F16F16:
    case IREE_AMD_UK_FLAG_PACK_TYPE_BF16BF16:
      return 2;
    case IREE_AMD_UK_FLAG_PACK_TYPE_I8I8:
      return 1;
    default:
      return 0;
  }
}

int oracle_pack(const iree_amd_uk_pack_params_t* p) {
  const int es = pack_elem_size(p->flags & IREE_AMD_UK_FLAG_PACK_TYPE_MASK);
  if (!es) return IREE_AMD_UK_STATUS_INVALID_ARGUMENT;
  if (p->flags & ~(0xFFu | IREE_AMD_UK_FLAG_PACK_TRANSPOSE_INNER |
                   IREE_AMD_UK_FLAG_PACK_TRANSPOSE_OUTER))
    return IREE_AMD_UK_STATUS_INVALID_ARGUMENT;
  if (p->out_stride1 != p->out_size2 * p->out_size3)
    return IREE_AMD_UK_STATUS_INVALID_ARGUMENT;
  if (p->in_size0 < 0 || p->in_size1 < 0 || p->out_size0 < 0 ||
      p->out_size1 < 0 || p->out_size2 < 0 || p->out_size3 < 0 ||
      p->in_stride0 < 0 || p->in_stride1 < 0 || p->out_stride0 < 0)
    return IREE_AMD_UK_STATUS_INVALID_ARGUMENT;
  /* Walk the destination in ITS OWN index order (d0,d1,d2,d3) and derive which
   * source coordinate each slot maps to; the transposes decide which of the
   * destination indices are the "row" pair and which the "column" pair. */
  const int t_outer = (p->flags & IREE_AMD_UK_FLAG_PACK_TRANSPOSE_OUTER) != 0;
  const int t_inner = (p->flags & IREE_AMD_UK_FLAG_PACK_TRANSPOSE_INNER) != 0;
  const int64_t tile_rows = t_inner ? p->out_size3 : p->out_size2;
  const int64_t tile_cols = t_inner ? p->out_size2 : p->out_size3;
  const int64_t outer_rows = t_outer ? p->out_size1 : p->out_size0;
  const int64_t outer_cols = t_outer ? p->out_size0 : p->out_size1;
  if (outer_rows * tile_rows < p->in_size0 || outer_cols * tile_cols < p->in_size1)
    return IREE_AMD_UK_STATUS_INVALID_ARGUMENT;
  if (!p->out_size0 || !p->out_size1 || !p->out_size2 || !p->out_size3) return 0;
  const char* in = (const char*)p->in_buffer;
  char* out = (char*)p->out_buffer;
  const uint64_t pad = p->padding_value; /* little-endian low bytes */
  for (int64_t d0 = 0; d0 < p->out_size0; ++d0)
    for (int64_t d1 = 0; d1 < p->out_size1; ++d1)
      for (int64_t d2 = 0; d2 < p->out_size2; ++d2)
        for (int64_t d3 = 0; d3 < p->out_size3; ++d3) {
          const int64_t orow = t_outer ? d1 : d0, ocol = t_outer ? d0 : d1;
          const int64_t trow = t_inner ? d3 : d2, tcol = t_inner ? d2 : d3;
          const int64_t r = orow * tile_rows + trow;
          const int64_t c = ocol * tile_cols + tcol;
          const int64_t dst = p->out_offset + d0 * p->out_stride0 +
                              d1 * p->out_stride1 + d2 * p->out_size3 + d3;
          if (r < p->in_size0 && c < p->in_size1) {
            const int64_t src = p->in_offset + r * p->in_stride0 + c * p->in_stride1;
            memcpy(out + dst * es, in + src * es, (size_t)es);
          } else {
            memcpy(out + dst * es, &pad, (size_t)es);
          }
        }
  return 0;
}

int oracle_unpack(const iree_amd_uk_unpack_params_t* p) {
  const uint32_t type = p->flags & IREE_AMD_UK_FLAG_UNPACK_TYPE_MASK;
  const int es = (type == IREE_AMD_UK_FLAG_PACK_TYPE_I8I8) ? 0 : pack_elem_size(type);
  if (!es) return IREE_AMD_UK_STATUS_INVALID_ARGUMENT;
  if (p->flags & ~(0xFFu | IREE_AMD_UK_FLAG_UNPACK_TRANSPOSE_INNER |
                   IREE_AMD_UK_FLAG_UNPACK_TRANSPOSE_OUTER))
    return IREE_AMD_UK_STATUS_INVALID_ARGUMENT;
  if (p->in_stride1 != p->in_size2 * p->in_size3)
    return IREE_AMD_UK_STATUS_INVALID_ARGUMENT;
  if (p->in_size0 < 0 || p->in_size1 < 0 || p->in_size2 < 0 || p->in_size3 < 0 ||
      p->out_size0 < 0 || p->out_size1 < 0 || p->in_stride0 < 0 ||
      p->out_stride0 < 0 || p->out_stride1 < 0)
    return IREE_AMD_UK_STATUS_INVALID_ARGUMENT;
  const int t_outer = (p->flags & IREE_AMD_UK_FLAG_UNPACK_TRANSPOSE_OUTER) != 0;
  const int t_inner = (p->flags & IREE_AMD_UK_FLAG_UNPACK_TRANSPOSE_INNER) != 0;
  const int64_t tile_rows = t_inner ? p->in_size3 : p->in_size2;
  const int64_t tile_cols = t_inner ? p->in_size2 : p->in_size3;
  const int64_t outer_rows = t_outer ? p->in_size1 : p->in_size0;
  const int64_t outer_cols = t_outer ? p->in_size0 : p->in_size1;
  if (outer_rows * tile_rows < p->out_size0 || outer_cols * tile_cols < p->out_size1)
    return IREE_AMD_UK_STATUS_INVALID_ARGUMENT;
  if (!p->out_size0 || !p->out_size1) return 0;
  const char* in = (const char*)p->in_buffer;
  char* out = (char*)p->out_buffer;
  /* Walk the DESTINATION (row-major) and locate each element in the tiles. */
  for (int64_t r = 0; r < p->out_size0; ++r)
    for (int64_t c = 0; c < p->out_size1; ++c) {
      const int64_t orow = r / tile_rows, trow = r % tile_rows;
      const int64_t ocol = c / tile_cols, tcol = c % tile_cols;
      const int64_t d0 = t_outer ? ocol : orow, d1 = t_outer ? orow : ocol;
      const int64_t d2 = t_inner ? tcol : trow, d3 = t_inner ? trow : tcol;
      const int64_t src = p->in_offset + d0 * p->in_stride0 + d1 * p->in_stride1 +
                          d2 * p->in_size3 + d3;
      const int64_t dst = p->out_offset + r * p->out_stride0 + c * p->out_stride1;
      memcpy(out + dst * es, in + src * es, (size_t)es);
    }
  return 0;
}

int oracle_query_role_tile(uint32_t flags, int M0, int N0, int K0,
                           int64_t* t0, int64_t* t1) {
  switch (flags & IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_MASK) {
    case IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_LHS:
      *t0 = M0, *t1 = K0;
      return 0;
    case IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_RHS:
      *t0 = N0, *t1 = K0;
      return 0;
    case IREE_AMD_UK_FLAG_QUERY_TILE_SIZES_OPERAND_ROLE_RESULT:
      *t0 = M0, *t1 = N0;
      return 0;
    default:
      return IREE_AMD_UK_STATUS_INVALID_ARGUMENT;
  }
}

/*---------------------------------------------------------------------------*
 * Row-major matmul, int4 dequant matmul, SiLU
 *---------------------------------------------------------------------------*/

int oracle_matmul_rowmajor(const void* a, const void* b, void* c, int64_t M,
                           int64_t N, int64_t K, uint32_t flags) {
  const uint32_t type = flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK;
  const int accf = (flags & IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE) != 0;
  if (type == IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32) {
    const int8_t* A = a;
    const int8_t* B = b;
    int32_t* C = c;
#pragma omp parallel for
    for (int64_t m = 0; m < M; ++m) {
      for (int64_t n = 0; n < N; ++n) {
        uint32_t acc = accf ? (uint32_t)C[m * N + n] : 0u;
        for (int64_t k = 0; k < K; ++k)
          acc += (uint32_t)((int32_t)A[m * K + k] * (int32_t)B[k * N + n]);
        C[m * N + n] = (int32_t)acc;
      }
    }
    return 0;
  }
  if (type == IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F32 ||
      type == IREE_AMD_UK_FLAG_MMT4D_TYPE_F32F32F32 ||
      type == IREE_AMD_UK_FLAG_MMT4D_TYPE_F8E4M3F8E4M3F32 ||
      type == IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16F32) {
    float* C = c;
#pragma omp parallel for
    for (int64_t m = 0; m < M; ++m) {
      for (int64_t n = 0; n < N; ++n) {
        double acc = accf ? (double)C[m * N + n] : 0.0;
        for (int64_t k = 0; k < K; ++k)
          acc += (double)load_flt(a, m * K + k, type, ORACLE_F16_IEEE) *
                 (double)load_flt(b, k * N + n, type, ORACLE_F16_IEEE);
        C[m * N + n] = (float)acc;
      }
    }
    return 0;
  }
  return IREE_AMD_UK_STATUS_UNIMPLEMENTED;
}

/* The reference matmul of the reference's end-to-end test runner: float
 * accumulation in f32 in k order starting from the accumulator operand (or 0),
 * the narrow result types rounded once at the end; i8 accumulates in i32. */
int oracle_e2e_reference_matmul(const void* a, const void* b, const void* acc,
                                void* c, int64_t M, int64_t N, int64_t K,
                                uint32_t flags) {
  const uint32_t type = flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK;
  if (type == IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32) {
    const int8_t* A = a;
    const int8_t* B = b;
    const int32_t* ACC = acc;
    int32_t* C = c;
#pragma omp parallel for
    for (int64_t m = 0; m < M; ++m)
      for (int64_t n = 0; n < N; ++n) {
        uint32_t sum = ACC ? (uint32_t)ACC[m * N + n] : 0u;
        for (int64_t k = 0; k < K; ++k)
          sum += (uint32_t)((int32_t)A[m * K + k] * (int32_t)B[k * N + n]);
        C[m * N + n] = (int32_t)sum;
      }
    return 0;
  }
  const int out_f16 = type == IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F16;
  const int out_bf16 = type == IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16BF16;
  if (!(out_f16 || out_bf16 || type == IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F32 ||
        type == IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16F32 ||
        type == IREE_AMD_UK_FLAG_MMT4D_TYPE_F32F32F32))
    return IREE_AMD_UK_STATUS_UNIMPLEMENTED;
#pragma omp parallel for
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      const int64_t o = m * N + n;
      float sum = 0.f;
      if (acc) {
        if (out_f16) sum = oracle_f16_to_f32(((const uint16_t*)acc)[o], ORACLE_F16_IEEE);
        else if (out_bf16) sum = oracle_bf16_to_f32(((const uint16_t*)acc)[o]);
        else sum = ((const float*)acc)[o];
      }
      for (int64_t k = 0; k < K; ++k) {
        /* (volatile: one rounding per multiply and per add, no contraction) */
        volatile float prod = load_flt(a, m * K + k, type, ORACLE_F16_IEEE) *
                              load_flt(b, k * N + n, type, ORACLE_F16_IEEE);
        sum += prod;
      }
      if (out_f16) ((uint16_t*)c)[o] = oracle_f32_to_f16(sum);
      else if (out_bf16) ((uint16_t*)c)[o] = oracle_f32_to_bf16(sum);
      else ((float*)c)[o] = sum;
    }
  return 0;
}

/* The pseudorandom stream of the reference's test tools: a Lehmer step whose
 * product is taken in 32-bit unsigned arithmetic (so it wraps before the
 * reduction), then value = state % range + min. Returns the final state. */
uint32_t oracle_e2e_pseudorandom_fill(uint32_t seed, int64_t n, int32_t min,
                                      int32_t max, int32_t* out) {
  uint32_t state = seed;
  const uint32_t range = (uint32_t)(max - min + 1);
  for (int64_t i = 0; i < n; ++i) {
    state = (uint32_t)(state * 48271u) % 2147483647u;
    out[i] = (int32_t)(state % range) + min;
  }
  return state;
}

int oracle_dequant_matmul_i4(const uint16_t* x, const uint8_t* w,
                             const uint16_t* scale, const void* zp,
                             uint16_t* out, int64_t M, int64_t N, int64_t K,
                             int64_t gs, int zp_is_u4) {
  if (gs <= 0 || K % gs || (K & 1)) return IREE_AMD_UK_STATUS_INVALID_ARGUMENT;
  const int64_t G = K / gs;
#pragma omp parallel for
  for (int64_t n = 0; n < N; ++n) {
    for (int64_t m = 0; m < M; ++m) {
      double acc = 0.0;
      for (int64_t g = 0; g < G; ++g) {
        const int64_t sg = n * G + g;
        const double s = oracle_f16_to_f32(scale[sg], ORACLE_F16_IEEE);
        double z;
        if (zp_is_u4) {
          uint8_t b = ((const uint8_t*)zp)[sg >> 1];
          z = (sg & 1) ? (b >> 4) : (b & 0xF);
        } else {
          z = oracle_f16_to_f32(((const uint16_t*)zp)[sg], ORACLE_F16_IEEE);
        }
        for (int64_t k = 0; k < gs; ++k) {
          const int64_t e = n * K + g * gs + k;
          const uint8_t b = w[e >> 1];
          const double q = (e & 1) ? (b >> 4) : (b & 0xF);
          const double xv = oracle_f16_to_f32(x[m * K + g * gs + k], ORACLE_F16_IEEE);
          acc += xv * ((q - z) * s);
        }
      }
      out[m * N + n] = f32_to_f16_ieee((float)acc);
    }
  }
  return 0;
}

/* The reassociated form of the same dispatch
 * (REF compiler/src/iree/compiler/GlobalOptimization/FuseDequantizationMatmul.cpp:
 * generateGroupMaxGeneric :398-415, generateScalesGeneric :419-441 with
 * (1 << (16 - 1)) - 1 = 32767, generateGroupSumsGeneric :445-461, the quantize
 * generic :483-492 (divf then fptosi), the integer matmul :539-562 (sext i16,
 * zext i4, i32 multiply-accumulate per group), and the final generic :622-633
 * (sitofp; * new scale; * scale; zp * scale; * group sum; subf; addf over the
 * groups in order)), in f32 as the pattern's float type: the activations are
 * widened from f16 first. "Introduces precision loss ... opt-in only"
 * (:746-748). fptosi truncates toward zero. A group of zeros has scale 0 and
 * 0/0 in the quantize step; the reference leaves that undefined, here the
 * group's quantised values are 0. */
int oracle_quantize_groups_i16(const uint16_t* x, int64_t M, int64_t K, int64_t gs,
                               int16_t* q, float* scale_x, float* group_sum) {
  if (gs <= 0 || K % gs) return IREE_AMD_UK_STATUS_INVALID_ARGUMENT;
  const int64_t G = K / gs;
  for (int64_t m = 0; m < M; ++m)
    for (int64_t g = 0; g < G; ++g) {
      const uint16_t* xs = x + m * K + g * gs;
      float mx = 0.0f, sum = 0.0f;
      for (int64_t k = 0; k < gs; ++k) {
        const float v = oracle_f16_to_f32(xs[k], ORACLE_F16_IEEE);
        const float a = fabsf(v);
        mx = a > mx ? a : mx;
        sum = sum + v;
      }
      const float sc = mx / 32767.0f;
      scale_x[m * G + g] = sc;
      group_sum[m * G + g] = sum;
      for (int64_t k = 0; k < gs; ++k) {
        const float v = oracle_f16_to_f32(xs[k], ORACLE_F16_IEEE);
        q[m * K + g * gs + k] = sc > 0.0f ? (int16_t)(v / sc) : (int16_t)0;
      }
    }
  return 0;
}

int oracle_dequant_matmul_i4_reassoc(const uint16_t* x, const uint8_t* w,
                                     const uint16_t* scale, const void* zp,
                                     uint16_t* out, int64_t M, int64_t N, int64_t K,
                                     int64_t gs, int zp_is_u4, int32_t* int_core) {
  if (gs <= 0 || K % gs || (K & 1)) return IREE_AMD_UK_STATUS_INVALID_ARGUMENT;
  const int64_t G = K / gs;
  int16_t* q = (int16_t*)malloc((size_t)(M * K > 0 ? M * K : 1) * sizeof(int16_t));
  float* sx = (float*)malloc((size_t)(M * G > 0 ? M * G : 1) * sizeof(float));
  float* gsum = (float*)malloc((size_t)(M * G > 0 ? M * G : 1) * sizeof(float));
  if (!q || !sx || !gsum) { free(q); free(sx); free(gsum); return 8; }
  const int st = oracle_quantize_groups_i16(x, M, K, gs, q, sx, gsum);
  if (st) { free(q); free(sx); free(gsum); return st; }
#pragma omp parallel for
  for (int64_t n = 0; n < N; ++n) {
    for (int64_t m = 0; m < M; ++m) {
      float acc_out = 0.0f;
      for (int64_t g = 0; g < G; ++g) {
        const int64_t sg = n * G + g;
        const float s = oracle_f16_to_f32(scale[sg], ORACLE_F16_IEEE);
        float z;
        if (zp_is_u4) {
          uint8_t b = ((const uint8_t*)zp)[sg >> 1];
          z = (float)((sg & 1) ? (b >> 4) : (b & 0xF));
        } else {
          z = oracle_f16_to_f32(((const uint16_t*)zp)[sg], ORACLE_F16_IEEE);
        }
        int32_t acc = 0;
        for (int64_t k = 0; k < gs; ++k) {
          const int64_t e = n * K + g * gs + k;
          const uint8_t b = w[e >> 1];
          const int32_t wv = (e & 1) ? (b >> 4) : (b & 0xF);
          acc += (int32_t)q[m * K + g * gs + k] * wv;
        }
        if (int_core) int_core[(m * N + n) * G + g] = acc;
        const float dq = (float)acc;
        const float r0 = dq * sx[m * G + g];
        const float r1 = r0 * s;
        const float z0 = z * s;
        const float z1 = z0 * gsum[m * G + g];
        const float res = r1 - z1;
        acc_out = res + acc_out;
      }
      out[m * N + n] = f32_to_f16_ieee(acc_out);
    }
  }
  free(q); free(sx); free(gsum);
  return 0;
}

double oracle_silu_mul(double g, double u) { return (g / (1.0 + exp(-g))) * u; }
