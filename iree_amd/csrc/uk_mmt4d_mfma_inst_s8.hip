// Kernel instances of the matrix-core mmt4d for one group of element types
// (see uk_mmt4d_mfma_launch.h).
#include "uk_mmt4d_mfma_launch.h"

namespace uk {

int launch_mfma_s8s8s32(const MfmaArgs& a, hipStream_t s) {
  // `a` counts K in steps of 32 (a.k0_div K tiles per step, a.tail_tiles left
  // over). The kernels run on the 16-row instruction, whose K-step is 64 bytes
  // of a row: less energy per operation than the 32-row one under the power
  // limit (4096^3: 63.7 -> 57.3 us; row-major left-hand side 69.5 -> 62.7,
  // whose lane quads then also load 64 contiguous bytes of a row).
  const int64_t tiles = (int64_t)a.ksteps * a.k0_div + a.tail_tiles;
  MfmaArgs b = a;
  b.k0_div = 2 * a.k0_div;
  b.ksteps = (int)(tiles / b.k0_div);
  b.tail_tiles = (int)(tiles % b.k0_div);
  // (a row-major left-hand side has no partial last step: a K in whole steps
  // of 32 but not of 64 stays on the 32-row instruction)
  if (a.k_slices <= 1 && !(a.lhs_row_major && b.tail_tiles)) return launch_cfg<S8Cfg16>(b, s);
  return launch_cfg<S8Cfg>(a, s);
}

}  // namespace uk
