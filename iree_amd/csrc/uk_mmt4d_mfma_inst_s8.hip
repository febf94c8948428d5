// Kernel instances of the matrix-core mmt4d for one group of element types
// (see uk_mmt4d_mfma_launch.h).
#include "uk_mmt4d_mfma_launch.h"

namespace uk {

int launch_mfma_s8s8s32(const MfmaArgs& a, hipStream_t s) { return launch_cfg<S8Cfg>(a, s); }

}  // namespace uk
