// One instantiation of the unrolled forward kernel: DiagCGproduct, 1 channel(s) of the first operand per thread.
#include "cg_unrolled_fwd_impl.h"

namespace gelib_hip {

int launch_unrolled_fwd_diag(const FwdArgs &a, int nblocks, hipStream_t s) {
  return launch_fwd_variant<true, 1>(a, nblocks, s);
}

}  // namespace gelib_hip
