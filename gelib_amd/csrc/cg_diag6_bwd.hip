// Instantiation of the lane-per-channel Diag backward kernel, l up to 6, one cell per wave.
#include "cg_diag6_impl.h"

namespace gelib_hip {

int launch_diag6_bwd_l6(const Diag6Args &a, hipStream_t s) { return launch_diag6_bwd_variant<kL6, false>(a, s); }

}  // namespace gelib_hip
