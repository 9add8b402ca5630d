// One instantiation of the unrolled backward kernels: CGproduct of operands up to l = 6, the part of the product above
// l = 6 (l = 7..12), power-of-two channel counts.  The triples up to l = 6 of such a product run on the instantiation in
// cg_unrolled_bwd_cg6l.hip first; this launch adds onto what that one wrote.
#include "cg_unrolled_bwd_impl.h"

namespace gelib_hip {

int launch_unrolled_bwd_cg6_hi(const BwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s) {
  return launch_bwd_variants<12, false, false, 6, false, 7>(a, nblocks, lds_bytes, s);
}

}  // namespace gelib_hip
