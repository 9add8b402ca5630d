// Fused product -> linear forward: the launch for the rows of pass 0 (see cg_linear_impl.h).
#include "cg_linear_impl.h"

namespace gelib_hip {

int launch_cg_linear_pass0(const LinArgs &a, long long nblocks, hipStream_t s) {
  return launch_cg_linear_pass_impl<0>(a, nblocks, s);
}

}  // namespace gelib_hip
