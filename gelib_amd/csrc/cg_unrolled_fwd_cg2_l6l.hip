// One instantiation of the unrolled forward kernel: CGproduct of operands up to l = 6, product capped at l = 6,
// 2 channels of the first operand per thread.
#include "cg_unrolled_fwd_impl.h"

namespace gelib_hip {

int launch_unrolled_fwd_cg2_l6l(const FwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s) {
  return launch_fwd_variant<6, false, 2, 6>(a, nblocks, lds_bytes, s);
}

}  // namespace gelib_hip
