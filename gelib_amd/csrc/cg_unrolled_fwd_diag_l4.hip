// One instantiation of the unrolled forward kernel: DiagCGproduct, 1 channel(s) of the first operand per thread,
// product l up to 4.
#include "cg_unrolled_fwd_impl.h"

namespace gelib_hip {

int launch_unrolled_fwd_diag_l4(const FwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s) {
  return launch_fwd_variant<4, true, 1>(a, nblocks, lds_bytes, s);
}

}  // namespace gelib_hip
