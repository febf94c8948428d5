// Kernel instances of the matrix-core mmt4d for one group of element types
// (see uk_mmt4d_mfma_launch.h).
#include "uk_mmt4d_mfma_launch.h"

namespace uk {

int launch_mfma_f8f8f32(const MfmaArgs& a, hipStream_t s) { return launch_cfg<F8Cfg>(a, s); }
int launch_mfma_silu_f8(const MfmaArgs& a, hipStream_t s) { return launch_cfg<F8Cfg, true>(a, s); }

}  // namespace uk
