// Kernel instances of the matrix-core mmt4d for one group of element types
// (see uk_mmt4d_mfma_launch.h).
#include "uk_mmt4d_mfma_launch.h"

namespace uk {

int launch_mfma_s8s8s32(const MfmaArgs& a, hipStream_t s) {
  // A row-major left-hand side with K0 = 16 and whole steps of 64: two
  // instructions per K-step, so that a lane quad loads 64 contiguous bytes.
  if (a.lhs_row_major && a.k0_div == 2 && a.tail_tiles == 0 && a.ksteps % 2 == 0 &&
      (a.k_slices <= 1 || a.slice_ksteps % 2 == 0)) {
    MfmaArgs b = a;
    b.ksteps = a.ksteps / 2;
    b.slice_ksteps = a.slice_ksteps / 2;
    b.k0_div = 4;
    return launch_cfg<S8Cfg2>(b, s);
  }
  return launch_cfg<S8Cfg>(a, s);
}

}  // namespace uk
