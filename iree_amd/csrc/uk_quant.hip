// Placeholder translation unit: int4 dequant-matmul and fp8 helpers.
#include "uk_common.h"
namespace uk {
int launch_dequant_matmul_i4(const void*, const void*, const void*, const void*, void*, int64_t,
                             int64_t, int64_t, int64_t, uint32_t, hipStream_t) {
  return fail(IREE_AMD_UK_STATUS_UNIMPLEMENTED, "dequant_matmul_i4: not built yet");
}
int launch_quantize_f16_to_f8e4m3(const void*, void*, int64_t, float, hipStream_t) {
  return fail(IREE_AMD_UK_STATUS_UNIMPLEMENTED, "quantize: not built yet");
}
int launch_silu_mul_quantize(const void*, const void*, void*, int64_t, int64_t, int64_t, float,
                             float, float, hipStream_t) {
  return fail(IREE_AMD_UK_STATUS_UNIMPLEMENTED, "silu_mul_quantize: not built yet");
}
}  // namespace uk
