// One instantiation of the unrolled forward kernel: CGproduct, 2 channel(s) of the first operand per thread.
#include "cg_unrolled_fwd_impl.h"

namespace gelib_hip {

int launch_unrolled_fwd_cg2(const FwdArgs &a, int nblocks, hipStream_t s) {
  return launch_fwd_variant<false, 2>(a, nblocks, s);
}

}  // namespace gelib_hip
