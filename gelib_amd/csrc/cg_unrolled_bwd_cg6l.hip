// One instantiation of the unrolled backward kernels: CGproduct of operands up to l = 6, product l up to 6,
// power-of-two channel counts (L = 6 vectors capped at maxl = 6).
#include "cg_unrolled_bwd_impl.h"

namespace gelib_hip {

int launch_unrolled_bwd_cg6_l6(const BwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s) {
  return launch_bwd_variants<6, false, false, 6>(a, nblocks, lds_bytes, s);
}

}  // namespace gelib_hip
