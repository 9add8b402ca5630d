// Kernels for any l up to GELIB_HIP_MAX_L with run-time m-loops (internal interface).
//
// Same preconditions as the unrolled small-l kernels (contiguous channels, leading dimensions that collapse into
// one cell index, destinations that do not broadcast), but nothing about l is fixed at compile time: a block
// stages the operands of its cells in LDS once, then walks every (l1,l2,l) triple of the product in one launch.
// They serve what the unrolled kernels do not cover (operand l above kLT, e.g. l = 6 or l = 10) and leave to the
// shape-agnostic kernels only strided channels, broadcast destinations and images too large for LDS.
#pragma once

#include <vector>

#include "cg_unrolled.h"

namespace gelib_hip {

// One (l1,l2,l) triple; lives in device memory next to the coefficient tables (read with scalar loads).
struct StagedTriple {
  int l1, l2, l;
  int n1, n2;
  int xi, yi, ri;   // positions in the x / y / product part lists of the kernel arguments
  int xoff, yoff;   // offsets (complex elements) of the operand parts inside one cell's packed x / y image
  int offs;         // first channel of this triple's block inside the product part
  int u;            // channel slots per cell: n1*n2, or n for Diag
  int log2_u;       // backward lane slots per cell, as a log2: n1p*n2p (Diag: n1p) with the channel counts rounded up
                    // to powers of two n1p, n2p (lanes beyond the real channels idle); -1 above 2^20
  int lg_n2p;       // log2(n2p)
  // Three compact copies of the coefficient table, each holding only the entries with |m1+m2| <= l, in the
  // order the corresponding loop nest visits them, so every kernel reads its coefficients as one stream:
  int cg_fwd;       // m ascending, then m1 ascending            (forward: one output row at a time)
  int cg_back0;     // m1 ascending, then m2 ascending           (gradient of x)
  int cg_back1;     // m2 ascending, then m1 ascending           (gradient of y)
};

// Part lists the kernels of this family take in their argument block (the block has to stay under 4 KB); vectors
// with more parts run on the shape-agnostic kernels.
constexpr int kStagedMaxParts = 16;
constexpr int kStagedMaxOutParts = 40;

struct StagedArgs {
  FastPart x[kStagedMaxParts], y[kStagedMaxParts], xg[kStagedMaxParts], yg[kStagedMaxParts];
  FastPart r[kStagedMaxOutParts];  // product (forward) or its gradient (backward)
  const StagedTriple *triples;
  const float *bank;
  // Striped backward kernels: (first, count, log2 of slots per cell) for every x part, then for every y part, then
  // the triple numbers ordered by x part, then ordered by y part; first indexes into the matching order list.
  const int *stripes;
  // Pair-wise backward kernel: (first triple, count, coefficient stream offset) per (x part, y part) pair.
  const int *pairs;
  int npairs;
  long long ncells;
  int ntriples;
  int nx, ny;
  int offs_add;   // extra channel offset (part-level calls)
  int accumulate;
  int xsize, ysize;  // complex elements of one cell's packed x / y image
  int cpb;           // cells per block
  int lds_coeffs;    // forward: floats of the coefficient stream staged in LDS behind the operands (0 = read from memory)
  int xrows[kStagedMaxParts], yrows[kStagedMaxParts];
};

// tile: adjacent output channels per lane (1, 2 or 4); threads: a multiple of 64 up to 1024
int launch_staged_fwd(const StagedArgs &a, bool diag, int tile, int threads, int nblocks, size_t lds_bytes,
                      hipStream_t s);
// cap: rows of g a lane keeps in registers (16 or 32); threads: 256, 512 or 1024 (1024 only with cap 16)
int launch_staged_bwd(const StagedArgs &a, bool diag, bool want_x, bool want_y, int cap, int threads, int nblocks,
                      size_t lds_bytes, hipStream_t s);

// role 0: gradient of x, 1: gradient of y; cap 16 or 32 (own 2l+1 must not exceed it)
int launch_staged_stripe(const StagedArgs &a, bool diag, int role, int cap, int nblocks, size_t lds_bytes,
                         hipStream_t s);

// both gradients from one pass over g, one (pair, 64 slots) unit at a time; cap 16 or 32
int launch_staged_pair_bwd(const StagedArgs &a, bool diag, bool want_x, bool want_y, int cap, int nblocks,
                           size_t lds_bytes, hipStream_t s);

// kind: 0 forward, 1 back0 (destination op.x), 2 back1 (destination op.y).  *used = 1 if a launch was made.
int staged_part(int kind, const PartOp &op, bool accumulate, hipStream_t s, int *used);
int staged_vec_fwd(const VecPlan &plan, const std::vector<const gelib_part_desc *> &r,
                   const std::vector<const gelib_part_desc *> &x, const std::vector<const gelib_part_desc *> &y,
                   bool accumulate, hipStream_t s, int *used);
int staged_vec_bwd(const VecPlan &plan, const std::vector<const gelib_part_desc *> &g,
                   const std::vector<const gelib_part_desc *> &x, const std::vector<const gelib_part_desc *> &y,
                   const std::vector<const gelib_part_desc *> &xg, const std::vector<const gelib_part_desc *> &yg,
                   bool accumulate, hipStream_t s, int *used);
int staged_set_option(const char *name, int value);

// Backward pass of a product of ONE x part with ONE y part, any l with l1 + l2 <= 21 (cg_onepair.hip).
int onepair_vec_bwd(const VecPlan &plan, const std::vector<const gelib_part_desc *> &g,
                    const std::vector<const gelib_part_desc *> &x, const std::vector<const gelib_part_desc *> &y,
                    const std::vector<const gelib_part_desc *> &xg, const std::vector<const gelib_part_desc *> &yg,
                    bool accumulate, hipStream_t s, int *used, bool dry_run = false);
int onepair_set_option(const char *name, int value);
// The same for 8 x 8 channels and l1, l2 <= 15 with the contraction over l on the matrix cores (cg_onepair_mfma.hip).
int onepair_mfma_vec_bwd(const VecPlan &plan, const std::vector<const gelib_part_desc *> &g,
                         const std::vector<const gelib_part_desc *> &x, const std::vector<const gelib_part_desc *> &y,
                         const std::vector<const gelib_part_desc *> &xg, const std::vector<const gelib_part_desc *> &yg,
                         bool accumulate, hipStream_t s, int *used);
// The forward pass of the same shapes on the matrix cores (the reduction over m1).
int onepair_mfma_vec_fwd(const VecPlan &plan, const std::vector<const gelib_part_desc *> &r,
                         const std::vector<const gelib_part_desc *> &x, const std::vector<const gelib_part_desc *> &y,
                         bool accumulate, hipStream_t s, int *used);
int onepair_mfma_set_option(const char *name, int value);  // "onepair_mfma", "onepair_mfma_fwd": 0 switches the kernel off

}  // namespace gelib_hip
