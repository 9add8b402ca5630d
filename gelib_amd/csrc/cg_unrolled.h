// Small-l kernels with every m-loop unrolled at compile time (internal interface).
//
// Covers operand parts with l1, l2 <= kLT whose channels are contiguous (channel stride 1) and whose leading
// dimensions (batch, grid0, grid1) collapse into one "cell" index.  One launch handles every (l1,l2,l) triple of
// an SO3vec product: the host builds, once per type signature, a table of (l1,l2) pairs with the channel offset
// and coefficient-table offset of each of their l, uploads it next to the concatenated coefficient tables, and
// keeps it cached on the device.
#pragma once

#include <vector>

#include "cg_common.h"

namespace gelib_hip {

constexpr int kLT = 4;                // largest operand l handled by the unrolled kernels
constexpr int kMaxDl = 2 * kLT + 1;   // most l values one (l1,l2) pair can produce
constexpr int kMaxPairs = (kLT + 1) * (kLT + 1);

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

// A part as the unrolled kernels see it: cells are sb apart, rows sm apart, channels contiguous.
struct FastPart {
  float2 *ptr;
  long long sb;
  int sm;
  int n;
};

// One (x part, y part) pair and the l it feeds; lives in device memory.
struct PairRec {
  int xi, yi, l1, l2, n1, n2;
  int ri[kMaxDl];    // product part index per dl = l - |l1-l2|, or -1 when that l is absent
  int offs[kMaxDl];  // first channel of the block in that part
  int cg[kMaxDl];    // offset (floats) of the triple's coefficient table from cg_base
  int cg_base;       // offset (floats) of this pair's tables in the bank that follows the pair array
  int cg_len;        // floats of coefficient tables belonging to this pair
  int xoff, yoff;    // offsets (complex elements) of the parts inside a per-cell packed x / y image (backward)
  int log2_u;        // log2 of the channel slots per cell (n1*n2, or n for Diag) when that is a power of two, else -1
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
