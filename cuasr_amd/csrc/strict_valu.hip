// Vector-ALU tile kernels for the floating-point semirings whose add is a
// comparison and whose mult is `multiplies` (min-times, max-times of
// include/cuasr/gemm/device/default_srgemm_configuration.h:161-218).  Their
// products can be -0.  The inner loop takes the hardware min / max and the
// epilogue restores the sign the reference's comparisons (functional.h:132,
// :172) give a zero result (valu_tile.h, ZERO_SIGN); that lookup and the
// epilogue's own add compare the way the reference does, so this file is built
// WITHOUT the no-NaN assumption the other tile files get, which would let the
// compiler turn those comparisons into min / max as well.
#include "valu_tile.h"

namespace cuasr_amd {

launch_fn find_valu_strict(int dtype, int add_op, int mult_op) {
  if (mult_op != kMultiplies) return nullptr;
  if (dtype == CUASR_AMD_F32 && add_op == kMinimum) return launch_valu_sized<float, kMinimum, kMultiplies, 8, 8, 32, 4, 4>;
  if (dtype == CUASR_AMD_F32 && add_op == kMaximum) return launch_valu_sized<float, kMaximum, kMultiplies, 8, 8, 32, 4, 4>;
  if (dtype == CUASR_AMD_F64 && add_op == kMinimum) return launch_valu_sized<double, kMinimum, kMultiplies, 8, 4, 16, 4, 4>;
  if (dtype == CUASR_AMD_F64 && add_op == kMaximum) return launch_valu_sized<double, kMaximum, kMultiplies, 8, 4, 16, 4, 4>;
  return nullptr;
}

}  // namespace cuasr_amd
