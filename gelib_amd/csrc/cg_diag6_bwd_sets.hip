// Instantiation of the lane-per-channel Diag backward kernel with the waves' sets of l2 fixed at compile time (every
// part of y up to l = 6 present), one cell per wave.
#include "cg_diag6_impl.h"

namespace gelib_hip {

int launch_diag6_bwd_l6_sets(const Diag6Args &a, hipStream_t s) { return launch_diag6_bwd_sets_variant<kL6, false>(a, s); }

}  // namespace gelib_hip
