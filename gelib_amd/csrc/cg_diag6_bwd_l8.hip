// Instantiation of the lane-per-channel Diag kernels for operand parts up to l = 4 and products up to l = 8 (the
// uncapped product of such vectors), one cell per wave.
#include "cg_diag6_impl.h"

namespace gelib_hip {

int launch_diag6_bwd_l8(const Diag6Args &a, hipStream_t s) { return launch_diag6_bwd_variant<8, false, 4>(a, s); }

}  // namespace gelib_hip
