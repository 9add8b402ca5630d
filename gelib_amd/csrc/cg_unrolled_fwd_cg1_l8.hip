// One instantiation of the unrolled forward kernel: CGproduct, 1 channel(s) of the first operand per thread,
// product l up to 8.
#include "cg_unrolled_fwd_impl.h"

namespace gelib_hip {

int launch_unrolled_fwd_cg1_l8(const FwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s) {
  return launch_fwd_variant<8, false, 1>(a, nblocks, lds_bytes, s);
}

}  // namespace gelib_hip
