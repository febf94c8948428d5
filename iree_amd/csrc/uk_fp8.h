// Device helpers shared by the fp8 element-wise kernels and the fused matmul
// epilogue: OCP e4m3fn encoding and the SiLU * up product.
#ifndef IREE_AMD_UK_FP8_H_
#define IREE_AMD_UK_FP8_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace uk {

// f32 -> OCP e4m3fn, round to nearest even, saturating at +-448 (NaN stays NaN).
__device__ __forceinline__ float clamp_e4m3(float x) {
  const float c = __builtin_fminf(__builtin_fmaxf(x, -448.0f), 448.0f);
  return x != x ? x : c;
}
// Four floats -> four e4m3 bytes (first value in the low byte).
__device__ __forceinline__ uint32_t pack4_e4m3(float a, float b, float c, float d) {
  int v = 0;
  v = __builtin_amdgcn_cvt_pk_fp8_f32(clamp_e4m3(a), clamp_e4m3(b), v, false);
  v = __builtin_amdgcn_cvt_pk_fp8_f32(clamp_e4m3(c), clamp_e4m3(d), v, true);
  return (uint32_t)v;
}

__device__ __forceinline__ float silu_mul(float g, float u) {
  // g / (1 + exp(-g)) * u; exp(-g) overflows to +inf for g < -88, giving -0.
  // (the reciprocal instruction, 1 ulp: a full division is 10 instructions per
  // element of an epilogue that runs while the matrix pipe idles)
  return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)) * u;
}

}  // namespace uk

#endif  // IREE_AMD_UK_FP8_H_
