// One instantiation of the single-triple backward kernel (cg_one_triple_bwd_impl.h): second operand of 32 channels,
// the triples whose code fits four waves per SIMD.
#include "cg_one_triple_bwd_impl.h"

namespace gelib_hip {

int launch_one_triple_bwd_k2_small(const BwdArgs &a, int l1, int l2, int l, int nblocks, size_t lds_bytes, hipStream_t s) {
  return launch_one_triple_k<2, true>(a, l1, l2, l, nblocks, lds_bytes, s);
}

}  // namespace gelib_hip
