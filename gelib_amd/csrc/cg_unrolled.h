// Small-l kernels with every m-loop unrolled at compile time (internal interface).
//
// Covers operand parts with l1, l2 <= kLT whose channels are contiguous (channel stride 1) and whose leading
// dimensions (batch, grid0, grid1) collapse into one "cell" index.  One launch handles every (l1,l2,l) triple of
// an SO3vec product: the host builds, once per type signature, a table of (l1,l2) pairs with the channel offset
// and coefficient-table offset of each of their l, uploads it next to the concatenated coefficient tables, and
// keeps it cached on the device.
#pragma once

#include <utility>
#include <vector>

#include "cg_common.h"

namespace gelib_hip {

constexpr int kLT = 4;                // largest operand l handled by the unrolled kernels
constexpr int kLTMax = 6;             // ... and by the one backward kernel built for operands up to l = 6 (product l <= 6)
constexpr int kMaxDl = 2 * kLTMax + 1;  // most l values one (l1,l2) pair can produce
constexpr int kMaxPairs = (kLTMax + 1) * (kLTMax + 1);  // most (x part, y part) pairs of one launch

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
  int log2_u;        // log2 of the lane slots per cell: n1p*n2p (Diag: n1p) with n1p, n2p the channel counts rounded up
                     // to powers of two; -1 when that exceeds 2^20
  int lg_n2p;        // log2 of n2p
  int rpc;           // runs of 64 lane slots per cell when a cell has 64 slots or more (else 0): n1p*n2p / 64, or
                     // n1*n2p / 64 (Diag: n1 / 64) when that is whole -- the channels of the first operand need no
                     // rounding up as long as a cell's slots fill whole runs
  unsigned rpc_magic;  // ceil(2^32 / rpc) for rpc > 1 (run / rpc = the high half of run * rpc_magic), else 0
  int rec_off;       // offset (floats) in the bank of the pair's step records (kernel for operands up to l = kLTMax), or -1
  int cost_rank;     // position of the pair when the pairs are sorted by falling cost (backward launches that deal the
                     // pairs of a cell to several blocks take every S-th of that order)
};

// Helpers shared by the kernel families that need contiguous channels and one cell index (cg_unrolled_plan.cpp).
bool collapse(const PartDev &p, const long long E[3], const long long own[3], long long *cell_stride);
// is_dest: the part is written; a destination that broadcasts over cells is refused (it needs a reduction)
bool to_fast(const PartDev &p, const long long E[3], const long long own[3], int n, bool is_dest, FastPart *out);
PartDev desc_to_dev(const gelib_part_desc *d, const long long E[3], long long own[3]);
// ln (optional) receives (l, n) of every part
bool lists_to_fast(const std::vector<const gelib_part_desc *> &ds, const long long E[3], bool is_dest,
                   std::vector<FastPart> *out, std::vector<std::pair<int, int>> *ln);
bool is_pow2(int v);
int ilog2(int v);

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

// Diag products of parts with l <= 6 and more than 32 channels, one lane per channel (cg_diag6.hip).
int diag6_vec_fwd(const VecPlan &plan, const std::vector<const gelib_part_desc *> &r,
                  const std::vector<const gelib_part_desc *> &x, const std::vector<const gelib_part_desc *> &y,
                  bool accumulate, hipStream_t s, int *used);
int diag6_vec_bwd(const VecPlan &plan, const std::vector<const gelib_part_desc *> &g,
                  const std::vector<const gelib_part_desc *> &x, const std::vector<const gelib_part_desc *> &y,
                  const std::vector<const gelib_part_desc *> &xg, const std::vector<const gelib_part_desc *> &yg,
                  bool accumulate, hipStream_t s, int *used);
// one triple; kind 0 forward, 1 gradient of x (x is the destination), 2 gradient of y; E = common leading extents
int diag6_part(int kind, const long long E[3], const gelib_part_desc *r, const gelib_part_desc *x,
               const gelib_part_desc *y, int l1, int l2, int l, int offs, bool accumulate, hipStream_t s, int *used);
int diag6_set_option(const char *name, int value);

}  // namespace gelib_hip
