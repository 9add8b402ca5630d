// One instantiation of the unrolled backward kernels: DiagCGproduct, product l up to 8, any channel counts (padded lane slots).
#include "cg_unrolled_bwd_impl.h"

namespace gelib_hip {

int launch_unrolled_bwd_diag8_pad(const BwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s) {
  return launch_bwd_variants<8, true, true>(a, nblocks, lds_bytes, s);
}

}  // namespace gelib_hip
