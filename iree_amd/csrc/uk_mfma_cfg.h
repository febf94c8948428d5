// MFMA instruction wrappers shared by the matmul kernels: one struct per
// element-type tuple and instruction shape giving the operand fragment type of
// one lane (16 bytes per 1 KiB operand block), the accumulator type of one
// kRows x kRows block and the instruction.
#ifndef IREE_AMD_UK_MFMA_CFG_H_
#define IREE_AMD_UK_MFMA_CFG_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace uk {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef int int4v __attribute__((ext_vector_type(4)));
typedef int int8v __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef int intx16 __attribute__((ext_vector_type(16)));
typedef int intx4 __attribute__((ext_vector_type(4)));

// kStepUs: measured time in microseconds of one K-step (the instruction's K
// extent) of a 256x256 macro tile with all compute units busy on MI355X; the
// launcher's estimates of absolute time start from it.
struct F16Cfg {
  static constexpr float kStepUs = 0.40f;
  static constexpr int kRows = 32;     // the instruction's block is kRows x kRows
  typedef half8 frag_t;
  typedef floatx16 acc_t;
  typedef float out_t;
  static constexpr int kElemBytes = 2;
  static constexpr int kMfmaK = 16;
  static constexpr int kSub = 1;   // 1 KiB pieces per operand block
  __device__ static acc_t mfma(frag_t a, frag_t b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};
struct BF16Cfg {
  static constexpr float kStepUs = 0.40f;
  static constexpr int kRows = 32;     // the instruction's block is kRows x kRows
  typedef bf16x8 frag_t;
  typedef floatx16 acc_t;
  typedef float out_t;
  static constexpr int kElemBytes = 2;
  static constexpr int kMfmaK = 16;
  static constexpr int kSub = 1;
  __device__ static acc_t mfma(frag_t a, frag_t b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
// The 16x16x32 shapes of the same types: half the rows, twice the K per
// instruction, the same 1 KiB operand block per fragment (lane l: row l % 16,
// k = 8 (l / 16) .. + 8). Measured on MI355X with N(0,1) data and no memory
// traffic at all, v_mfma_f32_16x16x32_f16 sustains 1.80-1.85 PFLOP/s where
// v_mfma_f32_32x32x16_f16 sustains 1.60: the matrix pipe is power-limited and
// the smaller block costs less energy per flop (with all-zero operands both
// run at 2.3-2.4).
struct F16Cfg16 {
  static constexpr float kStepUs = 0.69f;
  static constexpr int kRows = 16;
  typedef half8 frag_t;
  typedef floatx4 acc_t;
  typedef float out_t;
  static constexpr int kElemBytes = 2;
  static constexpr int kMfmaK = 32;
  static constexpr int kSub = 1;
  __device__ static acc_t mfma(frag_t a, frag_t b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};
struct BF16Cfg16 {
  static constexpr float kStepUs = 0.69f;
  static constexpr int kRows = 16;
  typedef bf16x8 frag_t;
  typedef floatx4 acc_t;
  typedef float out_t;
  static constexpr int kElemBytes = 2;
  static constexpr int kMfmaK = 32;
  static constexpr int kSub = 1;
  __device__ static acc_t mfma(frag_t a, frag_t b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
struct F16F16Cfg16 : F16Cfg16 {
  typedef _Float16 out_t;
};
struct BF16BF16Cfg16 : BF16Cfg16 {
  typedef __bf16 out_t;
};
// f16 / bf16 results: f32 accumulation, one rounding (to nearest even) when the
// accumulators are stored, which is the reference's arithmetic when
// IREE_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS is set
// (runtime/src/iree/builtins/ukernel/mmt4d_tile_generic.c:229-286, 289-376).
struct F16F16Cfg : F16Cfg {
  typedef _Float16 out_t;
};
struct BF16BF16Cfg : BF16Cfg {
  typedef __bf16 out_t;
};
// f32: v_mfma_f32_32x32x2_f32 takes one float per lane (row l % 32, k = l / 32).
// A lane's 16 bytes are 4 consecutive k of its row, so element e of lanes 0..31
// and element e of lanes 32..63 form the k pair of the e-th of four
// instructions; both operands pair the same way, so every k meets its partner.
struct F32Cfg {
  static constexpr float kStepUs = 1.75f;
  static constexpr int kRows = 32;     // the instruction's block is kRows x kRows
  typedef floatx4 frag_t;
  typedef floatx16 acc_t;
  typedef float out_t;
  static constexpr int kElemBytes = 4;
  static constexpr int kMfmaK = 8;
  static constexpr int kSub = 1;
  __device__ static acc_t mfma(frag_t a, frag_t b, acc_t c) {
#pragma unroll
    for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], c, 0, 0, 0);
    return c;
  }
};
struct S8Cfg {
  static constexpr float kStepUs = 0.38f;
  static constexpr int kRows = 32;     // the instruction's block is kRows x kRows
  typedef int4v frag_t;
  typedef intx16 acc_t;
  typedef int32_t out_t;
  static constexpr int kElemBytes = 1;
  static constexpr int kMfmaK = 32;
  static constexpr int kSub = 1;
  __device__ static acc_t mfma(frag_t a, frag_t b, acc_t c) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
  }
};
// The 16x16x64 shape of the same type: the f16 16-row layout (lane l: row
// l % 16, bytes 16 (l / 16) .. + 16 of a 64-byte K-step). With uniform random
// bytes and no memory traffic it sustains 4.16 POP/s where the 32x32x32 shape
// sustains 3.47 (both 4.92 on zeros): the smaller block costs less energy per
// operation, as with f16.
struct S8Cfg16 {
  static constexpr float kStepUs = 0.65f;
  static constexpr int kRows = 16;
  typedef int4v frag_t;
  typedef intx4 acc_t;
  typedef int32_t out_t;
  static constexpr int kElemBytes = 1;
  static constexpr int kMfmaK = 64;
  static constexpr int kSub = 1;
  __device__ static acc_t mfma(frag_t a, frag_t b, acc_t c) {
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
  }
};
struct F8Cfg {
  static constexpr float kStepUs = 0.86f;
  static constexpr int kRows = 32;     // the instruction's block is kRows x kRows
  typedef int8v frag_t;
  typedef floatx16 acc_t;
  typedef float out_t;
  static constexpr int kElemBytes = 1;
  static constexpr int kMfmaK = 64;
  static constexpr int kSub = 2;
  // formats 0 / 0: both operands e4m3; block scales 0x7F = 2^0. The scales are
  // per-lane register operands, and the instruction reads them from ALL lanes
  // whatever the execution mask: a kernel with divergent regions passes
  // `scales` from unit_scales(), called where every lane is active, because
  // the compiler is free to materialise the constant inside such a region,
  // where it reaches the active lanes only.
  __device__ static acc_t mfma(frag_t a, frag_t b, acc_t c, int scales = 0x7F7F7F7F) {
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, scales, 0, scales);
  }
  __device__ static int unit_scales() {
    int v;
    asm volatile("v_mov_b32 %0, 0x7f7f7f7f" : "=v"(v));
    return v;
  }
};

// Matrix-core instructions take their operands from all 64 lanes whatever the
// execution mask, but the compiler treats the fp8 one
// (v_mfma_scale_f32_32x32x64_f8f6f4) like per-lane arithmetic: when its result
// is only consumed inside a divergent region (stores of the lanes m0 < M0,
// say) it moves the instruction, and the per-lane selects and copies that
// prepare its operands, into that region, where those run for the active lanes
// only and the instruction then reads stale registers in all the others. This
// pins a result to the point where it is called, with every lane active: the
// empty volatile statement cannot move into a conditional block, and what
// produced its operand has to come before it. One element is enough, the
// instruction writes the whole block at once.
template <typename Acc>
__device__ __forceinline__ void keep_result_in_all_lanes(Acc& acc) {
  auto first = acc[0];
  asm volatile("" : "+v"(first));
  acc[0] = first;
}

// Configurations that are only built for a row-major left-hand side say so
// with a member kRowMajorLhsOnly.
template <typename Cfg, typename = void> struct RowMajorLhsOnly { static constexpr bool value = false; };
template <typename Cfg> struct RowMajorLhsOnly<Cfg, decltype((void)Cfg::kRowMajorLhsOnly)> {
  static constexpr bool value = Cfg::kRowMajorLhsOnly;
};

// The configuration that computes the same products with the accumulator type
// as result type (partial sums of a K split are kept in it).
template <typename Cfg> struct PartialSumCfg { typedef Cfg type; };
template <> struct PartialSumCfg<F16F16Cfg16> { typedef F16Cfg16 type; };
template <> struct PartialSumCfg<BF16BF16Cfg16> { typedef BF16Cfg16 type; };
template <> struct PartialSumCfg<F16F16Cfg> { typedef F16Cfg type; };
template <> struct PartialSumCfg<BF16BF16Cfg> { typedef BF16Cfg type; };

}  // namespace uk

#endif  // IREE_AMD_UK_MFMA_CFG_H_
