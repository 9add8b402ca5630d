// Instantiation of the lane-per-channel Diag forward kernel for the part of a product above l = 6: operand parts up to
// l = 6, product parts l = 7..12 (the parts up to l = 6 are a launch of the kernel in cg_diag6_fwd.hip), one cell and
// 64 channels per block.
#include "cg_diag6_impl.h"

namespace gelib_hip {

int launch_diag6_fwd_hi(const Diag6Args &a, hipStream_t s) { return launch_diag6_fwd_variant<2 * kL6, false, kL6, kL6 + 1>(a, s); }

}  // namespace gelib_hip
