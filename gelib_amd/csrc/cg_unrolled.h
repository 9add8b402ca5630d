// Small-l kernels with every m-loop unrolled at compile time (internal interface).
#pragma once

#include <vector>

#include "cg_common.h"

namespace gelib_hip {

struct VecTriple {
  int xi, yi, ri;  // indices into the l-sorted part lists
  int l1, l2, l;
  int offs;        // first channel of this triple's block inside the product part
  int nout;        // channels of the block
};

struct VecPlan {
  bool diag;
  long long E[3];
  std::vector<VecTriple> triples;  // reference order: l1 ascending, l2 ascending, l ascending
};

// kind: 0 forward, 1 back0 (destination op.x), 2 back1 (destination op.y).  *used = 1 if a launch was made.
int unrolled_part(int kind, const PartOp &op, bool accumulate, hipStream_t s, int *used);
int unrolled_vec_fwd(const VecPlan &plan, const std::vector<const gelib_part_desc *> &r,
                     const std::vector<const gelib_part_desc *> &x, const std::vector<const gelib_part_desc *> &y,
                     bool accumulate, hipStream_t s, int *used);
// xg / yg empty = that gradient is not wanted
int unrolled_vec_bwd(const VecPlan &plan, const std::vector<const gelib_part_desc *> &g,
                     const std::vector<const gelib_part_desc *> &x, const std::vector<const gelib_part_desc *> &y,
                     const std::vector<const gelib_part_desc *> &xg, const std::vector<const gelib_part_desc *> &yg,
                     bool accumulate, hipStream_t s, int *used);
int unrolled_set_option(const char *name, int value);

}  // namespace gelib_hip
