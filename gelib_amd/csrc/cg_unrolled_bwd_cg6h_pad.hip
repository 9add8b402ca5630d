// One instantiation of the unrolled backward kernels: CGproduct of operands up to l = 6, the part of the product above
// l = 6 (l = 7..12), channel counts that are not powers of two (padded lane slots).
#include "cg_unrolled_bwd_impl.h"

namespace gelib_hip {

int launch_unrolled_bwd_cg6_hi_pad(const BwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s) {
  return launch_bwd_variants<12, false, true, 6, false, 7>(a, nblocks, lds_bytes, s);
}

}  // namespace gelib_hip
