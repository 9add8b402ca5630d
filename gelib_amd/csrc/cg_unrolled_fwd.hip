// Dispatch of the unrolled forward kernels; the instantiations live in cg_unrolled_fwd_*.hip so that they
// compile in parallel.
#include "cg_unrolled_dev.h"

namespace gelib_hip {

int launch_unrolled_fwd_cg1_l4(const FwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_unrolled_fwd_cg1_l8(const FwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_unrolled_fwd_cg2_l4(const FwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_unrolled_fwd_cg2_l8(const FwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_unrolled_fwd_cg4_l4(const FwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_unrolled_fwd_cg4_l8(const FwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_unrolled_fwd_diag_l4(const FwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_unrolled_fwd_diag_l8(const FwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_unrolled_fwd_cg2_l6l(const FwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);

// Operands up to l = 4: every product, Diag or not.  Operands up to l = 6: CGproduct capped at l = 6 with two channels
// of the first operand per thread (one instantiation).
bool unrolled_fwd_takes(bool diag, int ti, int lcap, int lop) {
  if (lop <= kLT) return lcap <= 2 * kLT;
  return lop <= kLTMax && !diag && ti == 2 && lcap <= kLTMax;
}

// lcap: largest l present in the product; code for l above 4 is left out when the product is capped there
int launch_unrolled_fwd(const FwdArgs &a, bool diag, int ti, int lcap, int lop, int nblocks, size_t lds_bytes,
                        hipStream_t s) {
  if (nblocks <= 0) return GELIB_HIP_OK;
  if (lop > kLT) return launch_unrolled_fwd_cg2_l6l(a, nblocks, lds_bytes, s);
  const bool small = lcap <= kLT;
  if (diag) return small ? launch_unrolled_fwd_diag_l4(a, nblocks, lds_bytes, s) : launch_unrolled_fwd_diag_l8(a, nblocks, lds_bytes, s);
  if (ti == 4) return small ? launch_unrolled_fwd_cg4_l4(a, nblocks, lds_bytes, s) : launch_unrolled_fwd_cg4_l8(a, nblocks, lds_bytes, s);
  if (ti == 2) return small ? launch_unrolled_fwd_cg2_l4(a, nblocks, lds_bytes, s) : launch_unrolled_fwd_cg2_l8(a, nblocks, lds_bytes, s);
  return small ? launch_unrolled_fwd_cg1_l4(a, nblocks, lds_bytes, s) : launch_unrolled_fwd_cg1_l8(a, nblocks, lds_bytes, s);
}

}  // namespace gelib_hip
