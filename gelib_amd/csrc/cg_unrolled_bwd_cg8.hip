// One instantiation of the unrolled backward kernels: CGproduct, product l up to 8, power-of-two channel counts.
#include "cg_unrolled_bwd_impl.h"

namespace gelib_hip {

int launch_unrolled_bwd_cg8(const BwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s) {
  return launch_bwd_variants<8, false, false>(a, nblocks, lds_bytes, s);
}

}  // namespace gelib_hip
