// One instantiation of the unrolled forward kernel: CGproduct, 4 channel(s) of the first operand per thread.
#include "cg_unrolled_fwd_impl.h"

namespace gelib_hip {

int launch_unrolled_fwd_cg4(const FwdArgs &a, int nblocks, hipStream_t s) {
  return launch_fwd_variant<false, 4>(a, nblocks, s);
}

}  // namespace gelib_hip
