// Generic mmt4d kernel: any element type of the ABI, any M0/N0/K0, any strides
// and offsets. One thread owns one output element and walks the reduction in
// the order k (outer) then k0 (inner), multiply then add with no contraction,
// which is the order the reference's generic tile functions use
// (runtime/src/iree/builtins/ukernel/mmt4d_tile_generic.c:11-376). It exists for
// coverage and as the fallback behind ALLOW_GENERIC_FALLBACK_TILE_FUNCTION; the
// MFMA kernels in uk_mmt4d_mfma.hip are the fast path.
//
// 16-bit floats are decoded as IEEE (subnormals kept), like the reference's
// x86 tile functions (vcvtph2ps) and unlike its generic C path, which flushes
// f16 subnormals (common.h:685-686).
#include "uk_common.h"

#include <hip/hip_fp16.h>

namespace uk {
namespace {

struct GenericArgs {
  const void* lhs;
  const void* rhs;
  void* out;
  int64_t lhs_offset, lhs_stride0, rhs_offset, rhs_stride0, out_offset, out_stride0;
  int64_t M, N, K;
  int M0, N0, K0;
  int accumulate;
  int skip_rounding;
};

__device__ __forceinline__ float bf16_to_f32(uint16_t v) {
  return __uint_as_float((uint32_t)v << 16);
}
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x7FFF);  // quiet NaN, all mantissa bits
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
__device__ __forceinline__ float f16_to_f32(uint16_t v) {
  return __half2float(__ushort_as_half(v));
}
__device__ __forceinline__ uint16_t f32_to_f16(float f) {
  return __half_as_ushort(__float2half_rn(f));
}
// OCP e4m3fn: no infinities, S.1111.111 is NaN, subnormals kept.
__device__ __forceinline__ float f8e4m3_to_f32(uint8_t v) {
  const uint32_t s = (uint32_t)(v & 0x80) << 24;
  const uint32_t e = (v >> 3) & 0xF, m = v & 7;
  if (e == 15 && m == 7) return __uint_as_float(s | 0x7FFFFFFFu);
  if (e == 0) {
    float mag = (float)m * 0.001953125f;  // m * 2^-9
    return __uint_as_float(__float_as_uint(mag) | s);
  }
  return __uint_as_float(s | ((e + 120u) << 23) | (m << 20));
}

template <int TYPE>
struct Traits;

#define UK_INT_TRAITS(TYPE_, LHS_T, RHS_EXPR)                                  \
  template <>                                                                   \
  struct Traits<TYPE_> {                                                        \
    static constexpr bool kFloat = false;                                       \
    typedef int32_t acc_t;                                                      \
    __device__ static int32_t lhs(const void* b, int64_t i) {                   \
      return ((const LHS_T*)b)[i];                                              \
    }                                                                           \
    __device__ static int32_t rhs(const void* b, int64_t i) { RHS_EXPR; }       \
  };

UK_INT_TRAITS(IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32, int8_t, return ((const int8_t*)b)[i])
UK_INT_TRAITS(IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S16S32, int16_t, return ((const int16_t*)b)[i])
UK_INT_TRAITS(IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S8S32, int16_t, return ((const int8_t*)b)[i])
// 4-bit right-hand sides: element i is in byte i/2, even elements in the low
// nibble; u4 zero-extends, s4 sign-extends.
UK_INT_TRAITS(IREE_AMD_UK_FLAG_MMT4D_TYPE_S16U4S32, int16_t,
              uint8_t v = ((const uint8_t*)b)[i >> 1]; return (i & 1) ? (v >> 4) : (v & 0xF))
UK_INT_TRAITS(IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S4S32, int8_t,
              uint8_t v = ((const uint8_t*)b)[i >> 1]; int32_t n = (i & 1) ? (v >> 4) : (v & 0xF);
              return (n & 8) ? n - 16 : n)
#undef UK_INT_TRAITS

#define UK_FLT_TRAITS(TYPE_, LOAD_EXPR, OUT16, OUT_LOAD, OUT_STORE)             \
  template <>                                                                   \
  struct Traits<TYPE_> {                                                        \
    static constexpr bool kFloat = true;                                        \
    static constexpr bool kOut16 = OUT16;                                       \
    __device__ static float lhs(const void* b, int64_t i) { LOAD_EXPR; }        \
    __device__ static float rhs(const void* b, int64_t i) { LOAD_EXPR; }        \
    __device__ static float out_load(const void* b, int64_t i) { OUT_LOAD; }    \
    __device__ static void out_store(void* b, int64_t i, float v) { OUT_STORE; } \
  };

UK_FLT_TRAITS(IREE_AMD_UK_FLAG_MMT4D_TYPE_F32F32F32, return ((const float*)b)[i], false,
              return ((const float*)b)[i], ((float*)b)[i] = v)
UK_FLT_TRAITS(IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F32, return f16_to_f32(((const uint16_t*)b)[i]), false,
              return ((const float*)b)[i], ((float*)b)[i] = v)
UK_FLT_TRAITS(IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16F32, return bf16_to_f32(((const uint16_t*)b)[i]), false,
              return ((const float*)b)[i], ((float*)b)[i] = v)
UK_FLT_TRAITS(IREE_AMD_UK_FLAG_MMT4D_TYPE_F8E4M3F8E4M3F32, return f8e4m3_to_f32(((const uint8_t*)b)[i]), false,
              return ((const float*)b)[i], ((float*)b)[i] = v)
UK_FLT_TRAITS(IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F16, return f16_to_f32(((const uint16_t*)b)[i]), true,
              return f16_to_f32(((const uint16_t*)b)[i]), ((uint16_t*)b)[i] = f32_to_f16(v))
UK_FLT_TRAITS(IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16BF16, return bf16_to_f32(((const uint16_t*)b)[i]), true,
              return bf16_to_f32(((const uint16_t*)b)[i]), ((uint16_t*)b)[i] = f32_to_bf16(v))
#undef UK_FLT_TRAITS

template <int TYPE>
__global__ __launch_bounds__(256) void mmt4d_generic_kernel(GenericArgs a) {
  typedef Traits<TYPE> T;
  const int64_t tile_elems = (int64_t)a.M0 * a.N0;
  const int64_t total = a.M * a.N * tile_elems;
  const int64_t lhs_tile = (int64_t)a.M0 * a.K0, rhs_tile = (int64_t)a.N0 * a.K0;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t tile = idx / tile_elems;
    const int in_tile = (int)(idx - tile * tile_elems);
    const int64_t i = tile / a.N, j = tile - i * a.N;
    const int i0 = in_tile / a.N0, j0 = in_tile - i0 * a.N0;
    const int64_t o = a.out_offset + i * a.out_stride0 + j * tile_elems + in_tile;
    const int64_t lb = a.lhs_offset + i * a.lhs_stride0 + (int64_t)i0 * a.K0;
    const int64_t rb = a.rhs_offset + j * a.rhs_stride0 + (int64_t)j0 * a.K0;
    if constexpr (!T::kFloat) {
      uint32_t acc = a.accumulate ? (uint32_t)((const int32_t*)a.out)[o] : 0u;
      for (int64_t k = 0; k < a.K; ++k)
        for (int k0 = 0; k0 < a.K0; ++k0)
          acc += (uint32_t)(T::lhs(a.lhs, lb + k * lhs_tile + k0) *
                            T::rhs(a.rhs, rb + k * rhs_tile + k0));
      ((int32_t*)a.out)[o] = (int32_t)acc;
    } else {
      float acc = a.accumulate ? T::out_load(a.out, o) : 0.f;
      if (T::kOut16 && !a.skip_rounding) {
        // Accumulator lives in the 16-bit type: re-round after every step.
        for (int64_t k = 0; k < a.K; ++k)
          for (int k0 = 0; k0 < a.K0; ++k0) {
            float prod = __fmul_rn(T::lhs(a.lhs, lb + k * lhs_tile + k0),
                                   T::rhs(a.rhs, rb + k * rhs_tile + k0));
            float sum = __fadd_rn(acc, prod);
            if (TYPE == IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F16)
              acc = f16_to_f32(f32_to_f16(sum));
            else
              acc = bf16_to_f32(f32_to_bf16(sum));
          }
      } else {
        for (int64_t k = 0; k < a.K; ++k)
          for (int k0 = 0; k0 < a.K0; ++k0)
            acc = __fadd_rn(acc, __fmul_rn(T::lhs(a.lhs, lb + k * lhs_tile + k0),
                                           T::rhs(a.rhs, rb + k * rhs_tile + k0)));
      }
      T::out_store(a.out, o, acc);
    }
  }
}

template <int TYPE>
int launch(const GenericArgs& a, hipStream_t s) {
  const int64_t total = a.M * a.N * a.M0 * a.N0;
  int64_t blocks = ceil_div(total, 256);
  const int64_t max_blocks = (int64_t)device_cu_count() * 64;
  if (blocks > max_blocks) blocks = max_blocks;
  hipLaunchKernelGGL(mmt4d_generic_kernel<TYPE>, dim3((unsigned)blocks), dim3(256), 0, s, a);
  return check_hip(hipGetLastError(), "mmt4d_generic launch");
}

}  // namespace

int launch_mmt4d_generic(const iree_amd_uk_mmt4d_params_t& p, hipStream_t s) {
  GenericArgs a;
  a.lhs = p.lhs_buffer; a.rhs = p.rhs_buffer; a.out = p.out_buffer;
  a.lhs_offset = p.lhs_offset; a.lhs_stride0 = p.lhs_stride0;
  a.rhs_offset = p.rhs_offset; a.rhs_stride0 = p.rhs_stride0;
  a.out_offset = p.out_offset; a.out_stride0 = p.out_stride0;
  a.M = p.M; a.N = p.N; a.K = p.K; a.M0 = p.M0; a.N0 = p.N0; a.K0 = p.K0;
  a.accumulate = (p.flags & IREE_AMD_UK_FLAG_MMT4D_ACCUMULATE) != 0;
  a.skip_rounding = (p.flags & IREE_AMD_UK_FLAG_MMT4D_SKIP_INTERMEDIATE_ROUNDINGS) != 0;
  switch (p.flags & IREE_AMD_UK_FLAG_MMT4D_TYPE_MASK) {
#define UK_CASE(T) case T: return launch<T>(a, s);
    UK_CASE(IREE_AMD_UK_FLAG_MMT4D_TYPE_F32F32F32)
    UK_CASE(IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S8S32)
    UK_CASE(IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F32)
    UK_CASE(IREE_AMD_UK_FLAG_MMT4D_TYPE_F16F16F16)
    UK_CASE(IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16F32)
    UK_CASE(IREE_AMD_UK_FLAG_MMT4D_TYPE_BF16BF16BF16)
    UK_CASE(IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S16S32)
    UK_CASE(IREE_AMD_UK_FLAG_MMT4D_TYPE_S16U4S32)
    UK_CASE(IREE_AMD_UK_FLAG_MMT4D_TYPE_S16S8S32)
    UK_CASE(IREE_AMD_UK_FLAG_MMT4D_TYPE_S8S4S32)
    UK_CASE(IREE_AMD_UK_FLAG_MMT4D_TYPE_F8E4M3F8E4M3F32)
#undef UK_CASE
    default:
      return fail(IREE_AMD_UK_STATUS_INVALID_ARGUMENT, "mmt4d: unknown type");
  }
}

}  // namespace uk
