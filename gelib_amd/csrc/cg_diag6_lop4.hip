// Instantiations of the lane-per-channel Diag backward kernel for operand parts up to l = 4 with the product capped at
// l = 6 (the headline type's Diag product, and the l <= 6 part of its uncapped product): the images in LDS hold 25 rows
// of the y-gradient and 9 rows of x-gradient sums per wave instead of 49 and 13, so more blocks fit a compute unit
// (L=4, 64 channels, 131072 cells backward 7.3 -> 7.1 ms; L=2, 64 channels, 524288 cells uncapped 7.7 -> 7.05 ms).  The
// forward kernel built the same way is 2 to 4 % slower than the one for operands up to l = 6 and is not built.
#include "cg_diag6_impl.h"

namespace gelib_hip {

int launch_diag6_bwd_l6_lop4(const Diag6Args &a, hipStream_t s) { return launch_diag6_bwd_variant<kL6, false, 4>(a, s); }
int launch_diag6_bwd_l6_lop4_packed(const Diag6Args &a, hipStream_t s) { return launch_diag6_bwd_variant<kL6, true, 4>(a, s); }

}  // namespace gelib_hip
