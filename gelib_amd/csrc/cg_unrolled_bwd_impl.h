// Backward CG / DiagCG product for l1, l2 <= kLT (one instantiation: <= kLTMax): both gradients from one pass over g,
// all triples in one launch.
//
// Work split.  A block owns a few whole cells (one cell when a cell has >= 256 channel slots).  The operands x, y
// of those cells are staged once in LDS next to the coefficient bank.  For every (l1,l2) pair the flattened
// (cell, slot) space is cut into runs of 64 slots; the runs of all pairs are dealt to the four waves in turn.  In a run a lane owns one
// channel pair (i, j) of the gradient block: it reads g[m, i*n2+j] for every m (contiguous across the wave), forms
// C*g once per (m1,m2) and feeds two complex FMAs,
//     ax[m1] += (C g) conj(y[m2, j])        ay[m2] += (C g) conj(x[m1, i]),
// with all m-loops unrolled and x, y, ax, ay, g in registers.  ax is then summed over j inside aligned groups of
// n2 lanes (DPP butterflies), ay over i with butterflies at lane distance n2 and up (row swaps when n2 = 16), and
// the lanes that hold totals add them into the wave's private image of xg / yg in LDS: plain read-add-write in a fixed order, no atomics,
// no barrier.  After the last pair the four images are summed and written out in contiguous rows.
//
// Latency hiding.  A unit (pair, run, l) requests its rows of g and then computes on them; the kernel keeps its
// register count low enough for four waves per SIMD, and the other waves' arithmetic covers a wave's wait.  (A
// second register buffer holding the next unit's rows costs one wave of occupancy and the compiler does not keep
// those loads in flight across the control flow between units, so it lost to the plain form.)
#pragma once

// 1: every kernel for whole pairs reads its coefficients as step records (below), not only those for operands above
// kLT.  Measured on L=4, 16 channels, 32768 cells: backward 4.65 -> 4.4 ms capped at l = 4, 8.1 -> 7.3 ms uncapped.
#ifndef GELIB_BWD_RECORDS_ALL
#define GELIB_BWD_RECORDS_ALL 1
#endif

#include "cg_lane_sums.h"
#include "cg_unrolled_dev.h"

namespace gelib_hip {

namespace {

constexpr int cabs_(int a) { return a < 0 ? -a : a; }
constexpr int cmin_(int a, int b) { return a < b ? a : b; }
constexpr int kWaves = kBlock / kWave;
constexpr int pow2ceil_(int v) {
  int p = 1;
  while (p < v) p *= 2;
  return p;
}
// (m1,m2) steps of one row number m = m1 + m2, and steps of all row numbers below m (rows run from -ltop up)
constexpr int steps_of(int l1, int l2, int m) {
  const int lo = -l1 > m - l2 ? -l1 : m - l2, hi = l1 < m + l2 ? l1 : m + l2;
  return hi >= lo ? hi - lo + 1 : 0;
}
constexpr int steps_below(int l1, int l2, int ltop, int m) {
  int s = 0;
  for (int k = -ltop; k < m; k++) s += steps_of(l1, l2, k);
  return s;
}
// Step records: the coefficients of a step, one for every l of the pair that has a row m = m1 + m2 (l >= |m|, from lmin
// up), the steps one after the other in the order the kernel takes them.  Position of the first coefficient of step k
// of row number m:
constexpr int rec_pos(int l1, int l2, int lmin, int ltop, int m, int k) {
  int pos = 0;
  for (int mm = -ltop; mm <= m; mm++) {
    const int ma = mm < 0 ? -mm : mm;
    const int nv = ltop - (lmin > ma ? lmin : ma) + 1;  // coefficients per step of this row number
    pos += (mm < m ? steps_of(l1, l2, mm) : k) * nv;
  }
  return pos;
}

// All g, x, y pointers that the arithmetic loops dereference are typed as global memory, so the loads are
// global_load (vmcnt only) rather than flat_load (which also ties up the LDS counter).
typedef float v2f __attribute__((ext_vector_type(2)));
typedef const __attribute__((address_space(1))) v2f *GlobalRows;

// Coefficients are read through the constant address space: the address is the same for every lane, so the
// compiler fetches them with scalar loads into SGPRs and they cost neither vector registers nor LDS traffic.
typedef const __attribute__((address_space(4))) float *CoeffPtr;

// The gradient parts, indexed by their l (the host fills BwdArgs::g that way), copied out of the kernel arguments
// once so that the unrolled code can name them with compile-time indices.
template <int LCAP>
struct GParts {
  FastPart G[LCAP + 1];
};

typedef const __attribute__((address_space(4))) PairRec *PairPtr;

// Position of a lane in one run of 64 slots of a pair.
struct LanePos {
  int cell_local;  // cell inside the block
  int u;           // channel slot inside the cell
  bool live;
};

// rpc > 0: a cell has rpc runs of 64 slots (not necessarily a power of two of them); otherwise 2^log2_u < 64 slots.
__device__ __forceinline__ LanePos lane_pos(int run, int lane, int log2_u, int rpc, unsigned rpc_magic, int ncell) {
  LanePos q;
  if (rpc > 0) {  // uniform
    q.cell_local = rpc > 1 ? (int)__umulhi((unsigned)run, rpc_magic) : run;
    q.u = ((run - q.cell_local * rpc) << 6) + lane;
  } else {
    const int flat = (run << 6) + lane;
    q.cell_local = flat >> log2_u;
    q.u = flat & ((1 << log2_u) - 1);
  }
  q.live = q.cell_local < ncell;
  if (!q.live) q.cell_local = ncell - 1;  // dead lanes read valid memory and never store
  return q;
}

// One run of one pair, all of its l together.  For every row number m = m1 + m2 the lane reads g_l[m] of every l,
// contracts over l first,
//     Q[m1,m2] = sum_l C_l[m1,m2] g_l[m1+m2]          (real coefficient times complex: 2 FMA per term)
// and then feeds both gradients once per (m1,m2):  ax[m1] += Q conj(y[m2]),  ay[m2] += Q conj(x[m1]).
// That is 2 instructions per term plus 8 per (m1,m2) instead of 10 per term.  An l of the pair whose part is absent
// reads a row of zeros and a table of zeros (zrows, Zc) instead, so the code has no branches.
// PAD: channel counts are not all powers of two.  Lane slots are then n1p x n2p with the counts rounded up; a lane
// whose (i, j) lies beyond the real channels reads channel 0, has its g forced to zero and never writes.
// REC: the coefficients come from the pair's step records instead of its tables: one record per (m1,m2) step in the
// order the steps run, holding C_l[m1,m2] of every l of the pair (zero for an absent l), padded to a power of two.
// Sixteen floats of records are fetched by one scalar load, a group ahead of their use, into one of two register
// groups.  (Read from the tables, the coefficients of a step lie in up to seven places; the compiler merges the loads
// of neighbouring steps' entries into long ones issued far ahead of their use and spills their registers, and a wave
// waits for a load at every step once the tables outgrow the scalar cache.)  Used by the kernel for operands up to
// l = kLTMax (L=6, 8 channels, 16384 cells: 5.2 -> 4.6 ms, and 3.8 ms with the registers this frees: three waves per
// SIMD).  The kernels for operands up to l = 4 keep the tables: with records the product capped at l = 4 runs at the
// same speed and the uncapped one slower (7.8 -> 9.6 ms; its records are 16 floats, one load per step, waited for
// one step later).
// ONLY >= 0: the call has ONE triple, l = |L1 - L2| + ONLY (a part-level call, or a vector call on one-part vectors):
// the code for the other l of the pair is left out.  (The branch-free form reads rows of zeros and multiplies by
// tables of zeros for the l that are absent: for (2, 3) -> 4 with 32 x 32 channels that is 510 multiply-adds per lane
// and run where 350 are needed, and 24 row loads where 9 are.)
// LLO: the launch takes only the l from LLO up (a product that reaches above l = 6 with operands above l = 4 is taken
// in two launches, l <= 6 and l >= 7, each reading its own parts of g; the second adds onto the first).
template <int L1, int L2, int LCAP, bool DIAG, bool WX, bool WY, bool PAD, bool REC, int ONLY = -1, int LLO = 0>
__device__ __forceinline__ void pair_bwd(const GParts<LCAP> &gp, PairPtr pr, CoeffPtr Cs, CoeffPtr Zc, GlobalRows zrows,
                                         const float2 *xs, const float2 *ys, float2 *xacc, float2 *yacc, int xsize,
                                         int ysize, long long cell0, int offs_add, const LanePos q) {
  // the pair's tables are indexed by dl = l - |L1 - L2|; the first one used
  constexpr int DL0 = ONLY >= 0 ? ONLY : (LLO > cabs_(L1 - L2) ? LLO - cabs_(L1 - L2) : 0);
  constexpr int LMIN = cabs_(L1 - L2) + DL0;
  constexpr int LTOP = ONLY >= 0 ? LMIN : cmin_(L1 + L2, LCAP);
  if constexpr (LMIN > LCAP || LMIN > L1 + L2) return;  // no l of this pair can be present
  static_assert(!(REC && ONLY >= 0), "the step records hold every l of the pair");
  constexpr int NLP = LTOP - LMIN + 1;
  // scalar loads: the record sits in constant memory and the pointer is uniform
  const __attribute__((address_space(4))) PairRec &p = *pr;
  const int N1 = p.n1, N2 = p.n2;
  const int lg_n2 = DIAG ? 0 : p.lg_n2p;
  const int N2P = 1 << lg_n2;  // lanes per group that share i
  int i = DIAG ? q.u : (q.u >> lg_n2);
  int j = DIAG ? q.u : (q.u & (N2P - 1));
  const bool valid = !PAD || (i < N1 && (DIAG || j < N2));
  if (PAD && !valid) i = 0, j = 0;
  const int chan = DIAG ? i : (PAD ? i * N2 + j : q.u);  // the lane's channel inside the triple's block
  const int span = p.log2_u < 6 ? (1 << p.log2_u) : kWave;  // lanes of a run that belong to one cell
  const long long cell = cell0 + q.cell_local;

  float2 xv[2 * L1 + 1], yv[2 * L2 + 1], ax[2 * L1 + 1], ay[2 * L2 + 1];
  if (WY) {
    const float2 *xp = xs + q.cell_local * xsize + p.xoff + i;
#pragma unroll
    for (int m1 = 0; m1 <= 2 * L1; m1++) xv[m1] = xp[m1 * N1];
  }
  if (WX) {
    const float2 *yp = ys + q.cell_local * ysize + p.yoff + j;
#pragma unroll
    for (int m2 = 0; m2 <= 2 * L2; m2++) yv[m2] = yp[m2 * N2];
  }
  if (PAD && !valid) {
    // A lane beyond the real channels works on channel (0, 0) with operands of zero: whatever it reads of g (finite
    // wherever that channel's own lane sees finite values), it adds zeros to the sums it shares.
#pragma unroll
    for (int m1 = 0; m1 <= 2 * L1; m1++) xv[m1] = make_float2(0.f, 0.f);
#pragma unroll
    for (int m2 = 0; m2 <= 2 * L2; m2++) yv[m2] = make_float2(0.f, 0.f);
  }
#pragma unroll
  for (int m1 = 0; m1 <= 2 * L1; m1++) ax[m1] = make_float2(0.f, 0.f);
#pragma unroll
  for (int m2 = 0; m2 <= 2 * L2; m2++) ay[m2] = make_float2(0.f, 0.f);

  GlobalRows gptr[NLP];
  int gsm[NLP];
  CoeffPtr cl[NLP];
  static_for<NLP>([&](auto dl_c) __attribute__((always_inline)) {
    constexpr int dl = decltype(dl_c)::value;
    const bool present = p.ri[DL0 + dl] >= 0;
    const FastPart G = gp.G[LMIN + dl];
    gptr[dl] = present ? (GlobalRows)G.ptr + cell * G.sb + (p.offs[DL0 + dl] + offs_add + chan) : zrows;
    gsm[dl] = present ? G.sm : 0;
    cl[dl] = present ? Cs + p.cg[DL0 + dl] : Zc;
  });
  // Step records are fetched with scalar loads, kGroup floats at a time into one of two sets of scalar registers: the
  // next group is on its way while the steps of this one run.  Scalar loads return in any order, so every wait for
  // one is a wait for all: the fewer groups, the fewer waits (16 floats per group: 3.7 ms on the l <= 6 launch of
  // L=6, 8 channels, 16384 cells; 32 floats: 2.9 ms).
  constexpr int kGroup = 32;
  constexpr int NREC = rec_pos(L1, L2, LMIN, LTOP, LTOP, steps_of(L1, L2, LTOP));  // floats of all steps
  constexpr int NGROUPS = (NREC + kGroup - 1) / kGroup;
  const CoeffPtr recs = Cs - p.cg_base + (REC ? p.rec_off : 0);   // Cs is the bank plus cg_base
  float cb[2][kGroup];
  auto load_group = [&](auto gc, float(&dst)[kGroup]) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < kGroup; t++) dst[t] = recs[decltype(gc)::value * kGroup + t];
  };
  if constexpr (REC) load_group(std::integral_constant<int, 0>{}, cb[0]);
  // rows of one m at a time, the rows of the next m requested before the arithmetic of this one; the scheduling
  // barrier between steps keeps the compiler from hoisting every load of the pair to the top (twice the registers)
  auto load_m = [&](auto mc, float2(&dst)[NLP]) __attribute__((always_inline)) {
    constexpr int m = decltype(mc)::value - LTOP;
    static_for<NLP>([&](auto dl_c) __attribute__((always_inline)) {
      constexpr int dl = decltype(dl_c)::value;
      constexpr int L = LMIN + dl;
      if constexpr (L >= cabs_(m)) {
        const v2f t = gptr[dl][(m + L) * gsm[dl]];
        dst[dl] = make_float2(t.x, t.y);
      }
    });
  };
  // Rows of PF consecutive m are in flight at a time: all rows of the pair when there are at most kRowBudget of
  // them (the wave then waits once per pair, and 16 waves per compute unit keep enough bytes in flight to cover
  // the memory latency), otherwise as many m as fit the budget.  The kernels for l up to 8 hold more sums and are
  // near the register limit of three waves per SIMD already, so their budget is smaller.
  constexpr int kRowBudget =
      (LCAP <= 4 || ONLY >= 0) ? 32 : (LCAP == kLTMax || LLO > 0) ? ((L1 > kLT || L2 > kLT) ? 16 : 32) : 14;
  constexpr int ROWS = (LTOP + 1) * (LTOP + 1) - LMIN * LMIN;  // sum of 2l+1 over the l of the pair
  constexpr int PF = ROWS <= kRowBudget ? 2 * LTOP + 1 : (kRowBudget / NLP > 1 ? kRowBudget / NLP : 1);
  float2 gq[PF][NLP];
  static_for<PF>([&](auto kc) __attribute__((always_inline)) {
    if constexpr (kc.value <= 2 * LTOP) load_m(kc, gq[kc.value]);
  });
  static_for<2 * LTOP + 1>([&](auto mc) __attribute__((always_inline)) {
    constexpr int mi = decltype(mc)::value;
    constexpr int m = mi - LTOP;
    constexpr int MABS = cabs_(m);
    float2 gl[NLP];
#pragma unroll
    for (int k = 0; k < NLP; k++) gl[k] = gq[mi % PF][k];
    if constexpr (mi + PF <= 2 * LTOP) load_m(std::integral_constant<int, mi + PF>{}, gq[mi % PF]);
    constexpr int M1LO = (-L1 > m - L2) ? -L1 : m - L2;
    constexpr int M1HI = (L1 < m + L2) ? L1 : m + L2;
    constexpr int NP = M1HI - M1LO + 1;
    // each (m1,m2) runs as one short dependent chain, fenced from the next, so only a handful of values are live
    // at any time (left alone, the scheduler interleaves all chains of an m and doubles the register count)
    static_for<NP>([&](auto kc) __attribute__((always_inline)) {
      constexpr int m1 = M1LO + decltype(kc)::value;
      constexpr int m2 = m - m1;
      float qr = 0.f, qi = 0.f;
      constexpr int kk = decltype(kc)::value;
      constexpr int DLV = (LMIN > MABS ? LMIN : MABS) - LMIN;       // the first dl with a row m
      constexpr int P0 = rec_pos(L1, L2, LMIN, LTOP, m, kk);         // the step's first coefficient
      // the step before this one (none: -1)
      constexpr int PPREV = (mi == 0 && kk == 0) ? -kGroup
                            : (kk > 0 ? rec_pos(L1, L2, LMIN, LTOP, m, kk - 1)
                                      : rec_pos(L1, L2, LMIN, LTOP, m - 1, steps_of(L1, L2, m - 1) - 1));
      constexpr int grp = P0 / kGroup;
      static_for<NLP>([&](auto dl_c) __attribute__((always_inline)) {
        constexpr int dl = decltype(dl_c)::value;
        if constexpr (LMIN + dl >= MABS) {
          float c;
          if constexpr (REC) c = cb[((P0 + dl - DLV) / kGroup) & 1][(P0 + dl - DLV) % kGroup];
          else c = cl[dl][(m1 + L1) * (2 * L2 + 1) + (m2 + L2)];
          qr = fmaf(c, gl[dl].x, qr);
          qi = fmaf(c, gl[dl].y, qi);
        }
      });
      if constexpr (REC && grp != (PPREV < 0 ? -1 : PPREV / kGroup) && grp + 1 < NGROUPS) {
        // The first step that starts in a group requests the next one, into the registers of the group before (whose
        // last coefficient an earlier step has used: a step has at most 13 coefficients, a group 32), and only after
        // its own coefficients have been waited for.
        __builtin_amdgcn_sched_barrier(0);
        load_group(std::integral_constant<int, grp + 1>{}, cb[(grp + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (WX) {
        const float2 yc = yv[m2 + L2];
        ax[m1 + L1].x = fmaf(qr, yc.x, ax[m1 + L1].x);
        ax[m1 + L1].x = fmaf(qi, yc.y, ax[m1 + L1].x);
        ax[m1 + L1].y = fmaf(qi, yc.x, ax[m1 + L1].y);
        ax[m1 + L1].y = fmaf(-qr, yc.y, ax[m1 + L1].y);
      }
      if (WY) {
        const float2 xc = xv[m1 + L1];
        ay[m2 + L2].x = fmaf(qr, xc.x, ay[m2 + L2].x);
        ay[m2 + L2].x = fmaf(qi, xc.y, ay[m2 + L2].x);
        ay[m2 + L2].y = fmaf(qi, xc.x, ay[m2 + L2].y);
        ay[m2 + L2].y = fmaf(-qr, xc.y, ay[m2 + L2].y);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    __builtin_amdgcn_sched_barrier(0);
  });
  // pin the sums here: without this the optimiser moves the whole chain of ay updates down to its first use after
  // the ax part, keeping every Q alive until then
#pragma unroll
  for (int m1 = 0; m1 <= 2 * L1; m1++) asm volatile("" : "+v"(ax[m1].x), "+v"(ax[m1].y));
#pragma unroll
  for (int m2 = 0; m2 <= 2 * L2; m2++) asm volatile("" : "+v"(ay[m2].x), "+v"(ay[m2].y));

  if (WX) {
    // more than 64 channels of y: a run holds 64 of the lanes that share i, the other runs of the same i add their
    // sums into the image after it
    const int N2G = N2P < kWave ? N2P : kWave;
    if (!DIAG) group_sum(ax, N2G);
    if (q.live && valid && (DIAG || (j & (N2G - 1)) == 0)) {
      float2 *xa = xacc + q.cell_local * xsize + p.xoff + i;
#pragma unroll
      for (int m1 = 0; m1 <= 2 * L1; m1++) {
        float2 o = xa[m1 * N1];
        o.x += ax[m1].x;
        o.y += ax[m1].y;
        xa[m1 * N1] = o;
      }
    }
  }
  if (WY && !DIAG && N2P == 16 && span == kWave) {
    // four lanes of a run share j (one per 16-lane row): sum them four values at a time; row k of the wave then
    // holds value 4t + k, a value being one float of ay, and every lane adds its own into the image
    constexpr int NV = 2 * (2 * L2 + 1);
    const int row = (q.u >> 4) & 3, col = q.u & 15;
    float *ya = reinterpret_cast<float *>(yacc + q.cell_local * ysize + p.yoff);
    const bool writer = q.live && col < N2;
    static_for<(NV + 3) / 4>([&](auto tc) __attribute__((always_inline)) {
      constexpr int t = decltype(tc)::value;
      auto val = [&](auto kc) __attribute__((always_inline)) {
        constexpr int v = 4 * t + decltype(kc)::value;
        if constexpr (v < NV) return (v & 1) ? ay[v >> 1].y : ay[v >> 1].x;
        else return 0.f;
      };
      const float total = rows_sum4(val(std::integral_constant<int, 0>{}), val(std::integral_constant<int, 1>{}),
                                    val(std::integral_constant<int, 2>{}), val(std::integral_constant<int, 3>{}));
      const int v = 4 * t + row;  // float v of ay: row v / 2 of the part, real or imaginary
      if (writer && v < NV) ya[((v >> 1) * N2 + col) * 2 + (v & 1)] += total;
    });
  } else if (WY) {
    if (!DIAG) stride_sum(ay, N2P, span);
    if (q.live && valid && (DIAG || (q.u & (span - 1)) < N2P)) {
      float2 *ya = yacc + q.cell_local * ysize + p.yoff + j;
#pragma unroll
      for (int m2 = 0; m2 <= 2 * L2; m2++) {
        float2 o = ya[m2 * N2];
        o.x += ay[m2].x;
        o.y += ay[m2].y;
        ya[m2 * N2] = o;
      }
    }
  }
}

// Copies between memory and the packed per-cell LDS image of a part list (each part's rows contiguous).
// TO_LDS: stage operands.  Otherwise: sum the nsum per-wave images (fixed order) and write the gradient out.
template <bool TO_LDS>
__device__ __forceinline__ void copy_image(const FastPart (&parts)[kFastIn], const int (&rows)[kFastIn], int nparts,
                                           float2 *img, int img_size, long long cell0, int ncell, int nsum,
                                           int sum_stride, bool accumulate) {
  int off = 0;
  static_for<kFastIn>([&](auto kc) __attribute__((always_inline)) {
    constexpr int k = decltype(kc)::value;
    if (k < nparts) {
      const FastPart P = parts[k];
      const int per_cell = rows[k] * P.n;
      const int total = per_cell * ncell;
      for (int e = threadIdx.x; e < total; e += kBlock) {
        const int c = e / per_cell;
        const int r = e - c * per_cell;
        const int m = r / P.n;
        const int ch = r - m * P.n;
        float2 *gptr = P.ptr + (cell0 + c) * P.sb + m * P.sm + ch;
        float2 *lptr = img + c * img_size + off + r;
        if (TO_LDS) {
          *lptr = *gptr;
        } else {
          float2 v = lptr[0];
          for (int w = 1; w < nsum; w++) {
            const float2 t = lptr[w * sum_stride];
            v.x += t.x;
            v.y += t.y;
          }
          if (accumulate) {
            const float2 o = *gptr;
            v.x += o.x;
            v.y += o.y;
          }
          *gptr = v;
        }
      }
      off += per_cell;
    }
  });
}

// LT: largest operand l of the pairs the kernel has code for.
// The kernel for operands above kLT is asked to fit three waves per SIMD (168 registers): left alone it takes 169.
// ONE: the call has one triple (a.only_dl says which l of its pair).
template <int L1, int L2, int LCAP, bool DIAG, bool WX, bool WY, bool PAD>
__device__ __forceinline__ void pair_bwd_one(int only_dl, const GParts<LCAP> &gp, PairPtr pr, CoeffPtr Cs, CoeffPtr Zc,
                                             GlobalRows zrows, const float2 *xs, const float2 *ys, float2 *xacc,
                                             float2 *yacc, int xsize, int ysize, long long cell0, int offs_add,
                                             const LanePos q) {
  static_for<2 * cmin_(L1, L2) + 1>([&](auto dc) __attribute__((always_inline)) {
    constexpr int D = decltype(dc)::value;
    if (only_dl == D)  // uniform
      pair_bwd<L1, L2, LCAP, DIAG, WX, WY, PAD, false, D>(gp, pr, Cs, Zc, zrows, xs, ys, xacc, yacc, xsize, ysize, cell0,
                                                           offs_add, q);
  });
}

template <int LCAP, bool DIAG, bool WX, bool WY, bool PAD, int LT, bool ONE, int LLO = 0>
__global__ void __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(LT > kLT ? 3 : 1)))
unrolled_bwd_kernel(const BwdArgs a) {
  constexpr int KR = 2 * LCAP + 1;
  extern __shared__ float lds[];
  const int xsize = a.xsize, ysize = a.ysize, cpb = a.cells_per_block;
  float2 *xs = reinterpret_cast<float2 *>(lds);  // staged operands of the block's cells
  float2 *ys = xs + cpb * xsize;
  float2 *xacc_all = ys + cpb * ysize;                 // [wave][cell][xsize]
  float2 *yacc_all = xacc_all + kWaves * cpb * xsize;  // [wave][cell][ysize]

  const int nsplit = a.pair_split;  // > 1: this block takes every nsplit-th pair (by cost rank) of its cells
  const int split = nsplit > 1 ? (int)(blockIdx.x % nsplit) : 0;
  const long long cell0 = (long long)(nsplit > 1 ? blockIdx.x / nsplit : blockIdx.x) * cpb;
  const long long left = a.ncells - cell0;
  const int ncell = left < cpb ? (int)left : cpb;
  // readfirstlane tells the compiler the wave index is uniform, so everything derived from it (which pair, which
  // run) stays in scalar registers and branches on it are scalar branches
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & (kWave - 1);

  if (WY) copy_image<true>(a.x, a.xrows, a.nx, xs, xsize, cell0, ncell, 0, 0, false);
  if (WX) copy_image<true>(a.y, a.yrows, a.ny, ys, ysize, cell0, ncell, 0, 0, false);
  {
    const int nacc = kWaves * cpb * (xsize + ysize);
    for (int i = threadIdx.x; i < nacc; i += kBlock) xacc_all[i] = make_float2(0.f, 0.f);
  }
  __syncthreads();

  float2 *xacc = xacc_all + wave * cpb * xsize;
  float2 *yacc = yacc_all + wave * cpb * ysize;

  // The wave's visits: for each pair in turn, runs wave, wave+4, ... of the pair's cpb*U slots.
  const PairPtr pairs = (PairPtr)a.pairs;
  const int npairs = a.npairs, offs_add = a.offs_add, only_dl = a.only_dl;
  (void)only_dl;
  auto runs_of = [&](int k) { return pairs[k].rpc > 0 ? cpb * pairs[k].rpc : ((cpb << pairs[k].log2_u) + kWave - 1) >> 6; };
  GParts<LCAP> gp;
  static_for<LCAP + 1>([&](auto l) __attribute__((always_inline)) { gp.G[l.value] = a.g[l.value]; });
  const CoeffPtr Zc = (CoeffPtr)(a.bank + a.zero_off);    // a table of zeros and ...
  const GlobalRows zrows = (GlobalRows)(a.bank + a.zero_off);  // ... a row of zeros, for parts that are absent
  int dealt = 0;  // runs handed out so far: the runs of all pairs go round the waves, so that pairs with fewer runs
                  // than waves (few channels, few cells per block) do not leave the same waves idle every time
  for (int pidx = 0; pidx < npairs; pidx++) {
    const PairPtr p = pairs + pidx;
    if (nsplit > 1 && p->cost_rank % nsplit != split) continue;
    const int nruns = runs_of(pidx);
    CoeffPtr C = (CoeffPtr)(a.bank + p->cg_base);
    const int first = (wave - dealt) & (kWaves - 1);
    dealt += nruns;
    for (int run = first; run < nruns; run += kWaves) {
      const LanePos q = lane_pos(run, lane, p->log2_u, p->rpc, p->rpc_magic, ncell);
      switch (p->l1 * (kLTMax + 1) + p->l2) {
#define GELIB_CASE(A, B)                                                                                      \
  case A * (kLTMax + 1) + B:                                                                                  \
    if constexpr (A <= LT && B <= LT && A + B >= LLO) { /* the pair has an l the launch takes */              \
      if constexpr (ONE)                                                                                      \
        pair_bwd_one<A, B, LCAP, DIAG, WX, WY, PAD>(only_dl, gp, p, C, Zc, zrows, xs, ys, xacc, yacc, xsize, ysize,   \
                                                    cell0, offs_add, q);                                      \
      else                                                                                                    \
        pair_bwd<A, B, LCAP, DIAG, WX, WY, PAD, (LT > kLT || GELIB_BWD_RECORDS_ALL), -1, LLO>(gp, p, C, Zc, zrows, xs, ys, xacc, yacc, xsize,  \
                                                                       ysize, cell0, offs_add, q);            \
    }                                                                                                         \
    break;
#define GELIB_ROW(A) \
  GELIB_CASE(A, 0) GELIB_CASE(A, 1) GELIB_CASE(A, 2) GELIB_CASE(A, 3) GELIB_CASE(A, 4) GELIB_CASE(A, 5) GELIB_CASE(A, 6)
        GELIB_ROW(0) GELIB_ROW(1) GELIB_ROW(2) GELIB_ROW(3) GELIB_ROW(4) GELIB_ROW(5) GELIB_ROW(6)
#undef GELIB_ROW
#undef GELIB_CASE
        default: break;
      }
    }
  }

  __syncthreads();
  if (nsplit > 1) {
    // the sums of this block's pairs (the four wave images added in their order) go to the block's slice of the
    // partial images; unrolled_bwd_sum_splits_kernel adds the slices of a cell and writes the gradients
    auto park = [&](float2 *part, const float2 *acc, int size) {
      float2 *dst = part + ((long long)split * a.ncells + cell0) * size;
      for (int e = threadIdx.x; e < ncell * size; e += kBlock) {
        float2 v = acc[e];
        for (int w = 1; w < kWaves; w++) {
          const float2 t = acc[w * cpb * size + e];
          v.x += t.x;
          v.y += t.y;
        }
        dst[e] = v;
      }
    };
    if (WX) park(a.part_x, xacc_all, xsize);
    if (WY) park(a.part_y, yacc_all, ysize);
    return;
  }
  if (WX) copy_image<false>(a.xg, a.xrows, a.nx, xacc_all, xsize, cell0, ncell, kWaves, cpb * xsize, a.accumulate != 0);
  if (WY) copy_image<false>(a.yg, a.yrows, a.ny, yacc_all, ysize, cell0, ncell, kWaves, cpb * ysize, a.accumulate != 0);
}

template <int LCAP, bool DIAG, bool WX, bool WY, bool PAD, int LT, bool ONE, int LLO>
int launch_variant(const BwdArgs &a, int nblocks, size_t lds, hipStream_t s) {
  auto kern = unrolled_bwd_kernel<LCAP, DIAG, WX, WY, PAD, LT, ONE, LLO>;
  static bool attr_set = false;  // benign race: setting the attribute twice is harmless
  if (!attr_set) {
    GELIB_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      152 * 1024));  // dynamic LDS above the 64 KB default; 8 KB left for static use
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3(nblocks), dim3(kBlock), lds, s, a);
  GELIB_HIP_TRY(hipGetLastError());
  return GELIB_HIP_OK;
}

// want_x / want_y select which gradients are computed
template <int LCAP, bool DIAG, bool PAD, int LT = kLT, bool ONE = false, int LLO = 0>
int launch_bwd_variants(const BwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s) {
  static_assert(kLTMax == 6 && LT <= kLTMax, "the case table above lists l1, l2 = 0..6");
  const bool wx = a.want_x != 0, wy = a.want_y != 0;
  if (wx && wy) return launch_variant<LCAP, DIAG, true, true, PAD, LT, ONE, LLO>(a, nblocks, lds_bytes, s);
  if (wx) return launch_variant<LCAP, DIAG, true, false, PAD, LT, ONE, LLO>(a, nblocks, lds_bytes, s);
  return launch_variant<LCAP, DIAG, false, true, PAD, LT, ONE, LLO>(a, nblocks, lds_bytes, s);
}

}  // namespace

}  // namespace gelib_hip
