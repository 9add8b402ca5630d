// Forward CG / DiagCG product for l1, l2 <= kLT, all (l1,l2,l) triples of an SO3vec product in one launch.
//
// Work split: a block owns one (x part, y part) pair and a run of cells.  It first copies the two operand parts
// of its cells into LDS (the only loads from memory it ever waits for); after that its 256 threads sweep the
// flattened (cell, slot) space, a slot being one channel pair (i0, j).  A thread holds y[m2, j] and TI values
// x[m1, i0 + k*n1/TI] in registers, so one scaled value C*y[m2,j] feeds TI complex FMAs, and its TI results of a
// row lie n1/TI * n2 channels apart: every store instruction of a wave writes one contiguous 512-byte run of the
// product row.  The store stream is never interrupted by a wait on a load: stores and loads share one in-order
// counter on this hardware, so a load issued behind a burst of stores would not return before they have drained.
// All loops over l, m and m1 are unrolled at compile time; the coefficients are fetched with scalar loads.
#pragma once

#include "cg_unrolled_dev.h"

namespace gelib_hip {

namespace {

constexpr int cabs_(int a) { return a < 0 ? -a : a; }
constexpr int cmin_(int a, int b) { return a < b ? a : b; }

// Coefficients are read through the constant address space: the address is the same for every lane, so the
// compiler fetches them with scalar loads into SGPRs and they cost neither vector registers nor LDS traffic.
typedef const __attribute__((address_space(4))) float *CoeffPtr;
typedef const __attribute__((address_space(4))) PairRec *PairPtr;
typedef float v2f __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(1))) v2f *GlobalOut;  // product rows: global_store, not flat_store

// One (l1,l2,l) triple for one thread: rows m = -L..L of the block, TI channels each.
template <int L1, int L2, int L, int TI>
__device__ __forceinline__ void triple_fwd(const float2 (&xv)[TI][2 * L1 + 1], const float2 (&yv)[2 * L2 + 1],
                                           CoeffPtr C, GlobalOut rp, int sm, int kstride, bool accumulate,
                                           bool live) {
#pragma unroll
  for (int m = -L; m <= L; m++) {
    float2 acc[TI];
#pragma unroll
    for (int k = 0; k < TI; k++) acc[k] = make_float2(0.f, 0.f);
#pragma unroll
    for (int m1 = -L1; m1 <= L1; m1++) {
      const int m2 = m - m1;
      if (m2 >= -L2 && m2 <= L2) {
        const float c = C[(m1 + L1) * (2 * L2 + 1) + (m2 + L2)];
        const float cyr = c * yv[m2 + L2].x, cyi = c * yv[m2 + L2].y;
#pragma unroll
        for (int k = 0; k < TI; k++) {
          const float2 xk = xv[k][m1 + L1];
          acc[k].x = fmaf(xk.x, cyr, acc[k].x);
          acc[k].x = fmaf(-xk.y, cyi, acc[k].x);
          acc[k].y = fmaf(xk.x, cyi, acc[k].y);
          acc[k].y = fmaf(xk.y, cyr, acc[k].y);
        }
      }
    }
    if (live) {
      GlobalOut row = rp + (m + L) * sm;
#pragma unroll
      for (int k = 0; k < TI; k++) {
        v2f v;
        v.x = acc[k].x;
        v.y = acc[k].y;
        if (accumulate) v += row[k * kstride];
        row[k * kstride] = v;
      }
    }
  }
}

// The product parts, indexed by their l (the host fills FwdArgs::r that way), copied out of the kernel arguments
// once so that the unrolled code can name them with compile-time indices.
template <int LCAP>
struct RParts {
  FastPart R[LCAP + 1];
};

template <int L1, int L2, int LCAP, int TI, bool DIAG>
__device__ __forceinline__ void pair_fwd(const RParts<LCAP> &rp_all, PairPtr pr, CoeffPtr Cs, const float2 *xs,
                                         const float2 *ys, int offs_add, bool accumulate, long long cell, int dc,
                                         int u, bool live) {
  const __attribute__((address_space(4))) PairRec &p = *pr;
  const int N1 = p.n1, N2 = p.n2;
  int i0, j;
  if (DIAG) {
    i0 = u;
    j = u;
  } else {
    i0 = u / N2;
    j = u - i0 * N2;
  }
  const int istep = N1 / TI;  // the thread's k-th channel of x is i0 + k*istep
  const float2 *xp = xs + dc * (2 * L1 + 1) * N1 + i0;
  const float2 *yp = ys + dc * (2 * L2 + 1) * N2 + j;
  float2 xv[TI][2 * L1 + 1], yv[2 * L2 + 1];
#pragma unroll
  for (int m1 = 0; m1 <= 2 * L1; m1++)
#pragma unroll
    for (int k = 0; k < TI; k++) xv[k][m1] = xp[m1 * N1 + k * istep];
#pragma unroll
  for (int m2 = 0; m2 <= 2 * L2; m2++) yv[m2] = yp[m2 * N2];

  constexpr int LMIN = cabs_(L1 - L2);
  constexpr int NL = 2 * cmin_(L1, L2) + 1;
  const int kstride = DIAG ? 0 : istep * N2;
  static_for<NL>([&](auto dl_c) __attribute__((always_inline)) {
    constexpr int dl = decltype(dl_c)::value;
    constexpr int L = LMIN + dl;
    if constexpr (L <= LCAP) {
      if (p.ri[dl] >= 0) {
        const FastPart R = rp_all.R[L];
        GlobalOut rp = (GlobalOut)R.ptr + cell * R.sb + (p.offs[dl] + offs_add + u);
        triple_fwd<L1, L2, L, TI>(xv, yv, Cs + p.cg[dl], rp, R.sm, kstride, accumulate, live);
      }
    }
  });
}

// memory -> LDS copy of one operand part for the block's cells; rows become contiguous (row stride n)
__device__ __forceinline__ void stage_part(float2 *dst, const FastPart P, int rows, long long cell0, int ncell) {
  const int per_cell = rows * P.n;
  const int total = per_cell * ncell;
  for (int e = threadIdx.x; e < total; e += kBlock) {
    const int c = e / per_cell;
    const int r = e - c * per_cell;
    const int m = r / P.n;
    const int ch = r - m * P.n;
    const v2f t = ((const __attribute__((address_space(1))) v2f *)P.ptr)[(cell0 + c) * P.sb + m * P.sm + ch];
    dst[e] = make_float2(t.x, t.y);
  }
}

// LT: largest operand l of the pairs the kernel has code for.
template <int LCAP, bool DIAG, int TI, int LT>
__global__ void __launch_bounds__(kBlock) unrolled_fwd_kernel(const FwdArgs a) {
  extern __shared__ float2 lds_ops[];
  int pidx = 0, first = 0;
  const int per_tile = a.blocks_per_tile;
  const int tile_idx = (int)blockIdx.x / per_tile, in_tile = (int)blockIdx.x - tile_idx * per_tile;
  static_for<(LT + 1) * (LT + 1)>([&](auto k) __attribute__((always_inline)) {
    if (k.value > 0 && k.value < a.npairs && in_tile >= a.first_block[k.value]) {
      pidx = k.value;
      first = a.first_block[k.value];
    }
  });
  const PairPtr p = (PairPtr)a.pairs + pidx;
  const int cpb = pick_int(a.cpb, pidx);
  const long long tile_end = (tile_idx + 1) * a.tile < a.ncells ? (tile_idx + 1) * a.tile : a.ncells;
  const long long cell0 = tile_idx * a.tile + (long long)(in_tile - first) * cpb;
  const long long left = tile_end - cell0;  // <= 0 for the surplus blocks of a short last tile
  const int ncell = left < cpb ? (int)(left > 0 ? left : 0) : cpb;
  const int l1 = p->l1, l2 = p->l2, n1 = p->n1, n2 = p->n2;

  float2 *xs = lds_ops;
  float2 *ys = xs + cpb * (2 * l1 + 1) * n1;
  stage_part(xs, pick_part(a.x, p->xi), 2 * l1 + 1, cell0, ncell);
  stage_part(ys, pick_part(a.y, p->yi), 2 * l2 + 1, cell0, ncell);
  RParts<LCAP> rp_all;
  static_for<LCAP + 1>([&](auto l) __attribute__((always_inline)) { rp_all.R[l.value] = a.r[l.value]; });
  const int offs_add = a.offs_add;
  const bool accumulate = a.accumulate != 0;
  __syncthreads();

  const int U = DIAG ? n1 : (n1 / TI) * n2;
  const int slots = ncell * U;
  const CoeffPtr C = (CoeffPtr)(a.bank + p->cg_base);
  const int code = l1 * (kLTMax + 1) + l2;
  for (int w0 = 0; w0 < slots; w0 += kBlock) {
    const int w = w0 + threadIdx.x;
    const bool live = w < slots;
    const int wc = live ? w : slots - 1;
    const int dc = wc / U;
    const int u = wc - dc * U;
    const long long cell = cell0 + dc;
    switch (code) {
#define GELIB_CASE(A, B)                                                                                      \
  case A * (kLTMax + 1) + B:                                                                                  \
    if constexpr (A <= LT && B <= LT)                                                                         \
      pair_fwd<A, B, LCAP, TI, DIAG>(rp_all, p, C, xs, ys, offs_add, accumulate, cell, dc, u, live);          \
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

template <int LCAP, bool DIAG, int TI, int LT = kLT>
int launch_fwd_variant(const FwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s) {
  static_assert(kLTMax == 6 && LT <= kLTMax, "the case table above lists l1, l2 = 0..6");
  hipLaunchKernelGGL((unrolled_fwd_kernel<LCAP, DIAG, TI, LT>), dim3(nblocks), dim3(kBlock), lds_bytes, s, a);
  GELIB_HIP_TRY(hipGetLastError());
  return GELIB_HIP_OK;
}

}  // namespace

}  // namespace gelib_hip
