// One instantiation of the unrolled backward kernels: CGproduct calls with ONE triple (any l up to 8), power-of-two
// channel counts; only the code of that l of the pair runs.
#include "cg_unrolled_bwd_impl.h"

namespace gelib_hip {

int launch_unrolled_bwd_one(const BwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s) {
  return launch_bwd_variants<8, false, false, kLT, true>(a, nblocks, lds_bytes, s);
}

}  // namespace gelib_hip
