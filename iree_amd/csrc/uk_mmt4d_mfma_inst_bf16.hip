// Kernel instances of the matrix-core mmt4d for one group of element types
// (see uk_mmt4d_mfma_launch.h).
#include "uk_mmt4d_mfma_launch.h"

namespace uk {

int launch_mfma_bf16bf16f32(const MfmaArgs& a, hipStream_t s) { return launch_cfg<BF16Cfg16>(a, s); }
int launch_mfma_bf16bf16bf16(const MfmaArgs& a, hipStream_t s) { return launch_cfg<BF16BF16Cfg16>(a, s); }

}  // namespace uk
