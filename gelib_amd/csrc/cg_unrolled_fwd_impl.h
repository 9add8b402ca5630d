// Forward CG / DiagCG product for l1, l2 <= kLT, all (l1,l2,l) triples of an SO3vec product in one launch.
//
// Work split: a block owns one (x part, y part) pair and a run of cells; its 256 threads cover the flattened
// (cell, slot) space, a slot being one channel pair (i0, j).  Each thread keeps its operands in registers --
// y[m2, j] and TI values x[m1, i0 + k*n1/TI] -- so one scaled value C*y[m2,j] feeds TI complex FMAs, and the
// TI results of a row are n1/TI * n2 channels apart: every store instruction of a wave writes one contiguous
// 512-byte run of the product row.  All loops over l, m and m1 are unrolled at compile time; the coefficient
// tables of the block's pair sit in LDS and are read at immediate offsets.
#pragma once

#include "cg_unrolled_dev.h"

namespace gelib_hip {

namespace {

constexpr int cabs_(int a) { return a < 0 ? -a : a; }
constexpr int cmin_(int a, int b) { return a < b ? a : b; }

// One (l1,l2,l) triple for one thread: rows m = -L..L of the block, TI channels each.
template <int L1, int L2, int L, int TI>
__device__ __forceinline__ void triple_fwd(const float2 (&xv)[TI][2 * L1 + 1], const float2 (&yv)[2 * L2 + 1],
                                           const float *__restrict__ C, float2 *__restrict__ rp, int sm, int kstride,
                                           bool accumulate, bool live) {
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
      float2 *row = rp + (m + L) * sm;
#pragma unroll
      for (int k = 0; k < TI; k++) {
        float2 v = acc[k];
        if (accumulate) {
          const float2 o = row[k * kstride];
          v.x += o.x;
          v.y += o.y;
        }
        row[k * kstride] = v;
      }
    }
  }
}

// The block's view of its pair: operand parts and the product part of each l, picked out of the kernel
// arguments once per block.
struct PairParts {
  FastPart X, Y;
  FastPart R[kMaxDl];
};

template <int L1, int L2, int TI, bool DIAG>
__device__ __forceinline__ void pair_fwd(const PairParts &pp, const PairRec &p, const float *Cs, int offs_add,
                                         bool accumulate, long long cell, int u, bool live) {
  const FastPart X = pp.X;
  const FastPart Y = pp.Y;
  int i0, j;
  if (DIAG) {
    i0 = u;
    j = u;
  } else {
    i0 = u / p.n2;
    j = u - i0 * p.n2;
  }
  const int istep = p.n1 / TI;  // the thread's k-th channel of x is i0 + k*istep
  const float2 *xp = X.ptr + cell * X.sb + i0;
  const float2 *yp = Y.ptr + cell * Y.sb + j;
  float2 xv[TI][2 * L1 + 1], yv[2 * L2 + 1];
#pragma unroll
  for (int m1 = 0; m1 <= 2 * L1; m1++)
#pragma unroll
    for (int k = 0; k < TI; k++) xv[k][m1] = xp[m1 * X.sm + k * istep];
#pragma unroll
  for (int m2 = 0; m2 <= 2 * L2; m2++) yv[m2] = yp[m2 * Y.sm];

  constexpr int LMIN = cabs_(L1 - L2);
  constexpr int NL = 2 * cmin_(L1, L2) + 1;
  const int kstride = DIAG ? 0 : istep * p.n2;
  static_for<NL>([&](auto dl_c) __attribute__((always_inline)) {
    constexpr int dl = decltype(dl_c)::value;
    constexpr int L = LMIN + dl;
    if (p.ri[dl] >= 0) {
      const FastPart R = pp.R[dl];
      float2 *rp = R.ptr + cell * R.sb + (p.offs[dl] + offs_add + u);
      triple_fwd<L1, L2, L, TI>(xv, yv, Cs + p.cg[dl], rp, R.sm, kstride, accumulate, live);
    }
  });
}

template <bool DIAG, int TI>
__global__ void __launch_bounds__(kBlock) unrolled_fwd_kernel(const FwdArgs a) {
  __shared__ float Cs[kMaxDl * (2 * kLT + 1) * (2 * kLT + 1)];
  int pidx = 0, first = 0;
  static_for<kMaxPairs>([&](auto k) __attribute__((always_inline)) {
    if (k.value > 0 && k.value < a.npairs && (int)blockIdx.x >= a.first_block[k.value]) {
      pidx = k.value;
      first = a.first_block[k.value];
    }
  });
  const PairRec &p = a.pairs[pidx];
  for (int i = threadIdx.x; i < p.cg_len; i += kBlock) Cs[i] = a.bank[p.cg_base + i];
  __syncthreads();

  PairParts pp;
  pp.X = pick_part(a.x, p.xi);
  pp.Y = pick_part(a.y, p.yi);
  static_for<kMaxDl>([&](auto d) __attribute__((always_inline)) { pp.R[d.value] = pick_part(a.r, p.ri[d.value]); });
  const int offs_add = a.offs_add;
  const bool accumulate = a.accumulate != 0;
  const int cpb = pick_int(a.cpb, pidx);
  const long long cell0 = (long long)((int)blockIdx.x - first) * cpb;
  const long long left = a.ncells - cell0;
  const int ncell = left < cpb ? (int)left : cpb;
  const int U = DIAG ? p.n1 : (p.n1 / TI) * p.n2;
  const int slots = ncell * U;
  const int code = p.l1 * (kLT + 1) + p.l2;
  for (int w0 = 0; w0 < slots; w0 += kBlock) {
    const int w = w0 + threadIdx.x;
    const bool live = w < slots;
    const int wc = live ? w : slots - 1;
    const int dc = wc / U;
    const int u = wc - dc * U;
    const long long cell = cell0 + dc;
    switch (code) {
#define GELIB_CASE(A, B) \
  case A * (kLT + 1) + B: pair_fwd<A, B, TI, DIAG>(pp, p, Cs, offs_add, accumulate, cell, u, live); break;
#define GELIB_ROW(A) GELIB_CASE(A, 0) GELIB_CASE(A, 1) GELIB_CASE(A, 2) GELIB_CASE(A, 3) GELIB_CASE(A, 4)
      GELIB_ROW(0) GELIB_ROW(1) GELIB_ROW(2) GELIB_ROW(3) GELIB_ROW(4)
#undef GELIB_ROW
#undef GELIB_CASE
      default: break;
    }
  }
}

template <bool DIAG, int TI>
int launch_fwd_variant(const FwdArgs &a, int nblocks, hipStream_t s) {
  static_assert(kLT == 4, "the case table above lists l1, l2 = 0..4");
  hipLaunchKernelGGL((unrolled_fwd_kernel<DIAG, TI>), dim3(nblocks), dim3(kBlock), 0, s, a);
  GELIB_HIP_TRY(hipGetLastError());
  return GELIB_HIP_OK;
}

}  // namespace

}  // namespace gelib_hip
