// Instantiation of the lane-per-channel Diag forward kernel, l up to 6, several cells per wave (32 channels or fewer).
#include "cg_diag6_impl.h"

namespace gelib_hip {

int launch_diag6_fwd_l6_packed(const Diag6Args &a, hipStream_t s) { return launch_diag6_fwd_variant<kL6, true>(a, s); }

}  // namespace gelib_hip
