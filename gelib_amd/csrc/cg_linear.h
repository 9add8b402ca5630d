// Fused SO3vec CGproduct -> per-l channel mixing, forward (internal interface; kernels in cg_linear.hip).
#pragma once

#include <vector>

#include "cg_unrolled.h"

namespace gelib_hip {

constexpr int kLinL = 4;         // largest l of operands and product the fused kernel takes
constexpr int kLinMaxN = 16;     // most channels of an operand part
constexpr int kLinMaxOut = 16;   // most output channels of a product part
constexpr int kLinCells = 32;    // cells per block: the rows of one matrix-core tile

// Bytes of workspace: the re-packed matrices of a product with tau[l] channels in part l (l = 0..kLinL) and a copy of
// the first operand (x_elems_per_cell complex numbers per cell) transposed per group of kLinCells cells.
size_t cg_linear_workspace_bytes(const long long tau[kLinL + 1], long long x_elems_per_cell, long long ncells);

// out_l[cell, m, :] (+)= P_l[cell, m, :] W_l with P = CGproduct(x, y) never stored.  w[k] belongs to r[k] (both l-sorted):
// (tau_l, n_out_l) complex, row-major, device memory.  *used = 0 when the shapes are not ones the kernel takes (nothing
// has been launched then).  Returns 0, 10 (HIP call failed) or 13 (workspace missing, misaligned or too small).
int cg_linear_fwd(const VecPlan &plan, const std::vector<const gelib_part_desc *> &r,
                  const std::vector<const gelib_part_desc *> &x, const std::vector<const gelib_part_desc *> &y,
                  const std::vector<const float2 *> &w, bool accumulate, void *ws, size_t ws_bytes, hipStream_t s,
                  int *used);

}  // namespace gelib_hip
