#include "cg_unrolled.h"

namespace gelib_hip {

int unrolled_part(int, const PartOp &, bool, hipStream_t, int *used) {
  *used = 0;
  return GELIB_HIP_OK;
}
int unrolled_vec_fwd(const VecPlan &, const std::vector<const gelib_part_desc *> &,
                     const std::vector<const gelib_part_desc *> &, const std::vector<const gelib_part_desc *> &, bool,
                     hipStream_t, int *used) {
  *used = 0;
  return GELIB_HIP_OK;
}
int unrolled_vec_bwd(const VecPlan &, const std::vector<const gelib_part_desc *> &,
                     const std::vector<const gelib_part_desc *> &, const std::vector<const gelib_part_desc *> &,
                     const std::vector<const gelib_part_desc *> &, const std::vector<const gelib_part_desc *> &, bool,
                     hipStream_t, int *used) {
  *used = 0;
  return GELIB_HIP_OK;
}
int unrolled_set_option(const char *, int) { return GELIB_HIP_ERR_ARG; }

}  // namespace gelib_hip
