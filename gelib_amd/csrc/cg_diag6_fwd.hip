// Instantiation of the lane-per-channel Diag forward kernel, l up to 6, one cell per wave.
#include "cg_diag6_impl.h"

namespace gelib_hip {

int launch_diag6_fwd_l6(const Diag6Args &a, hipStream_t s) { return launch_diag6_fwd_variant<kL6, false>(a, s); }

}  // namespace gelib_hip
