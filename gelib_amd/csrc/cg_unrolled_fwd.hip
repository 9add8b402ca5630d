// Dispatch of the unrolled forward kernels; the instantiations live in cg_unrolled_fwd_{cg1,cg2,cg4,diag}.hip so
// that they compile in parallel.
#include "cg_unrolled_dev.h"

namespace gelib_hip {

int launch_unrolled_fwd_cg1(const FwdArgs &a, int nblocks, hipStream_t s);
int launch_unrolled_fwd_cg2(const FwdArgs &a, int nblocks, hipStream_t s);
int launch_unrolled_fwd_cg4(const FwdArgs &a, int nblocks, hipStream_t s);
int launch_unrolled_fwd_diag(const FwdArgs &a, int nblocks, hipStream_t s);

int launch_unrolled_fwd(const FwdArgs &a, bool diag, int ti, int nblocks, hipStream_t s) {
  if (nblocks <= 0) return GELIB_HIP_OK;
  if (diag) return launch_unrolled_fwd_diag(a, nblocks, s);
  if (ti == 4) return launch_unrolled_fwd_cg4(a, nblocks, s);
  if (ti == 2) return launch_unrolled_fwd_cg2(a, nblocks, s);
  return launch_unrolled_fwd_cg1(a, nblocks, s);
}

}  // namespace gelib_hip
