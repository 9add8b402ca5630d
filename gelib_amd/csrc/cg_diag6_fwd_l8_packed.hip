// Instantiation of the lane-per-channel Diag kernels for operand parts up to l = 4 and products up to l = 8 (the
// uncapped product of such vectors), several cells per wave.
#include "cg_diag6_impl.h"

namespace gelib_hip {

int launch_diag6_fwd_l8_packed(const Diag6Args &a, hipStream_t s) { return launch_diag6_fwd_variant<8, true, 4>(a, s); }

}  // namespace gelib_hip
