// One instantiation of the unrolled backward kernels: CGproduct of operands up to l = 6, product capped at l = 6,
// channel counts that are not all powers of two (lane slots rounded up, the lanes beyond the real channels idle).
#include "cg_unrolled_bwd_impl.h"

namespace gelib_hip {

int launch_unrolled_bwd_cg6_l6_pad(const BwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s) {
  return launch_bwd_variants<6, false, true, 6>(a, nblocks, lds_bytes, s);
}

}  // namespace gelib_hip
