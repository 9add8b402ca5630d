// Both gradients of ONE (l1, l2, l) triple of a CGproduct -- a part-level call (SO3/SO3part.hpp:223-257), or the
// vector-level backward on one-part vectors, which is what SO3part.CGproduct's backward runs -- for a second operand of
// 16 K channels, K = 1 or 2, and a first operand of at least 16 (a power of two), l1, l2 <= 4, in launches with
// enough cells to give every wave whole cells.
//
// The kernel is bound by the vector unit (8 multiply-adds per term are what the mathematics needs, 10 with the
// coefficient), so what counts is every instruction that is not one of them.  Against the general kernel
// (cg_unrolled_bwd_impl.h, lane = one channel pair (i, j), sums over 32 lanes per run of 64 slots):
//   * lane = (i, j / K) and K neighbouring channels j of the second operand: the x-gradient's sum over j starts
//     inside the lane, and what is left is a sum over the 16 lanes of a row (four DPP steps, no shuffles through LDS);
//   * a lane keeps its K channels j for all the runs of a cell: y is read from LDS once per cell, the y-gradient sums
//     stay in registers across the wave's runs and are added over the four rows of the wave once per cell;
//   * a wave takes whole cells: every element of either gradient is formed by one wave, nothing is summed over waves,
//     and the waves of a block never wait for each other (no block barrier: a wave stages its cell's operands in its own
//     piece of LDS and writes its gradients out from there).
// One pass over g, fixed order of additions, no atomics.
#pragma once

#include "cg_unrolled_bwd_impl.h"

namespace gelib_hip {

namespace {

// Registers a body needs, roughly: y, the y-gradient sums and the rows of g per channel slot, x and the x-gradient sums.
// The bodies that fit four waves per SIMD (128 registers) are built into one kernel, the others into a second one, so
// that the large ones do not set the occupancy of the small ones.
constexpr bool one_triple_small(int l1, int l2, int l, int k) {
  return k * (4 * (2 * l2 + 1) + 2 * (2 * l + 1)) + 5 * (2 * l1 + 1) <= 120;
}

typedef float v4f __attribute__((ext_vector_type(4)));
typedef const __attribute__((address_space(1))) v4f *GlobalRows4;

template <int L1, int L2, int D, bool WX, bool WY, int K>
__device__ __forceinline__ void one_triple_cell(const BwdArgs &a, PairPtr pr, const float2 *xs, const float2 *ys,
                                                float2 *ximg, float2 *yimg, long long cell, int lane) {
  constexpr int L = cabs_(L1 - L2) + D;
  if constexpr (L > L1 + L2) return;
  constexpr int R1 = 2 * L1 + 1, R2 = 2 * L2 + 1, RL = 2 * L + 1;
  const __attribute__((address_space(4))) PairRec &p = *pr;
  const int N1 = p.n1, N2 = p.n2;
  const FastPart G = a.g[L];
  const CoeffPtr C = (CoeffPtr)(a.bank + p.cg_base + p.cg[D]);
  const int isub = lane >> 4, jc = lane & 15;

  float2 yv[K][R2], ay[K][R2];
  if (WX) {
#pragma unroll
    for (int k = 0; k < K; k++)
#pragma unroll
      for (int m2 = 0; m2 < R2; m2++) yv[k][m2] = ys[m2 * N2 + K * jc + k];
  }
#pragma unroll
  for (int k = 0; k < K; k++)
#pragma unroll
    for (int m2 = 0; m2 < R2; m2++) ay[k][m2] = make_float2(0.f, 0.f);
  const GlobalRows gcell = (GlobalRows)G.ptr + cell * G.sb + (p.offs[D] + a.offs_add + K * jc);

  for (int run = 0; run < (N1 >> 2); run++) {
    const int i = run * 4 + isub;
    // One product of every term enters with a minus sign.  Negating Q per term would cost an instruction per term; the
    // x-gradient keeps those products in sums of their own (axm, subtracted at the end), the y-gradient multiplies by
    // a negated copy of Im x made once per run.
    float2 xv[R1], ax[R1];
    float nxi[R1], axm[R1];
    if (WY) {
#pragma unroll
      for (int m1 = 0; m1 < R1; m1++) {
        xv[m1] = xs[m1 * N1 + i];
        nxi[m1] = -xv[m1].y;
        asm volatile("" : "+v"(nxi[m1]));
      }
    }
    const GlobalRows gp = gcell + i * N2;
    v2f g[K][RL];
    // the lane's K channels are neighbours: one load of 8 K bytes per row
#pragma unroll
    for (int r = 0; r < RL; r++) {
      if constexpr (K == 2) {
        const v4f t = *reinterpret_cast<GlobalRows4>(gp + r * G.sm);
        g[0][r] = v2f{t.x, t.y};
        g[1][r] = v2f{t.z, t.w};
      } else {
        g[0][r] = gp[r * G.sm];
      }
    }
#pragma unroll
    for (int m1 = 0; m1 < R1; m1++) ax[m1] = make_float2(0.f, 0.f), axm[m1] = 0.f;

    static_for<RL>([&](auto mc) __attribute__((always_inline)) {
      constexpr int m = decltype(mc)::value - L;
      constexpr int M1LO = (-L1 > m - L2) ? -L1 : m - L2;
      constexpr int M1HI = (L1 < m + L2) ? L1 : m + L2;
      static_for<(M1HI >= M1LO ? M1HI - M1LO + 1 : 0)>([&](auto kc) __attribute__((always_inline)) {
        constexpr int m1 = M1LO + decltype(kc)::value;
        constexpr int m2 = m - m1;
        const float cf = C[(m1 + L1) * R2 + (m2 + L2)];
#pragma unroll
        for (int k = 0; k < K; k++) {
          const float qr = cf * g[k][m + L].x, qi = cf * g[k][m + L].y;
          if (WX) {
            const float2 yc = yv[k][m2 + L2];
            ax[m1 + L1].x = fmaf(qr, yc.x, ax[m1 + L1].x);
            ax[m1 + L1].x = fmaf(qi, yc.y, ax[m1 + L1].x);
            ax[m1 + L1].y = fmaf(qi, yc.x, ax[m1 + L1].y);
            axm[m1 + L1] = fmaf(qr, yc.y, axm[m1 + L1]);
          }
          if (WY) {
            const float2 xc = xv[m1 + L1];
            ay[k][m2 + L2].x = fmaf(qr, xc.x, ay[k][m2 + L2].x);
            ay[k][m2 + L2].x = fmaf(qi, xc.y, ay[k][m2 + L2].x);
            ay[k][m2 + L2].y = fmaf(qi, xc.x, ay[k][m2 + L2].y);
            ay[k][m2 + L2].y = fmaf(qr, nxi[m1 + L1], ay[k][m2 + L2].y);
          }
        }
        __builtin_amdgcn_sched_barrier(0);  // one short chain at a time: the sums are the only long-lived values
      });
    });

    // pin the sums here: otherwise the optimiser moves the chain of ay updates below the store of the x-gradient,
    // keeping every Q of the run alive until then
#pragma unroll
    for (int m1 = 0; m1 < R1; m1++) {
      asm volatile("" : "+v"(ax[m1].x), "+v"(ax[m1].y), "+v"(axm[m1]));
      ax[m1].y -= axm[m1];
    }
#pragma unroll
    for (int k = 0; k < K; k++)
#pragma unroll
      for (int m2 = 0; m2 < R2; m2++) asm volatile("" : "+v"(ay[k][m2].x), "+v"(ay[k][m2].y));
    if (WX) {
      group_sum(ax, 16);  // every lane of the row ends with the totals; lane jc of the row stores row jc of the part
      float2 mine = ax[0];
#pragma unroll
      for (int m1 = 1; m1 < R1; m1++)
        if (jc == m1) mine = ax[m1];
      if (jc < R1) ximg[jc * N1 + i] = mine;
    }
  }

  if (WY) {
    // sum over the four rows of the wave (the four i of a run), four floats at a time: row r of the wave receives the
    // total of float 4 t + r, float v = ((m2 K + k) 2 + component)
    constexpr int NV = 2 * K * R2;
    const int row = lane >> 4;
    float *yi = reinterpret_cast<float *>(yimg);
    static_for<(NV + 3) / 4>([&](auto tc) __attribute__((always_inline)) {
      constexpr int t = decltype(tc)::value;
      auto val = [&](auto kc) __attribute__((always_inline)) {
        constexpr int v = 4 * t + decltype(kc)::value;
        if constexpr (v < NV) {
          constexpr int k = (v >> 1) % K, m2 = (v >> 1) / K;
          return (v & 1) ? ay[k][m2].y : ay[k][m2].x;
        } else {
          return 0.f;
        }
      };
      const float total = rows_sum4(val(std::integral_constant<int, 0>{}), val(std::integral_constant<int, 1>{}),
                                    val(std::integral_constant<int, 2>{}), val(std::integral_constant<int, 3>{}));
      const int v = 4 * t + row;
      const int k = (v >> 1) % K, m2 = (v >> 1) / K;
      if (v < NV) yi[(m2 * N2 + K * jc + k) * 2 + (v & 1)] = total;
    });
  }
}

// One part between memory and a wave's LDS image of it (rows contiguous); the channel count is a power of two.
// Done by ONE wave for itself: the wave's LDS operations execute in order, so no block barrier is involved.
template <bool TO_LDS>
__device__ __forceinline__ void wave_copy_part(const FastPart P, int rows, float2 *img, long long cell, int lane,
                                               bool accumulate) {
  const int lg = 31 - __builtin_clz(P.n), total = rows << lg;
  float2 *base = P.ptr + cell * P.sb;
  for (int e = lane; e < total; e += kWave) {
    float2 *gptr = base + (e >> lg) * P.sm + (e & (P.n - 1));
    if (TO_LDS) {
      img[e] = *gptr;
    } else {
      float2 v = img[e];
      if (accumulate) {
        const float2 o = *gptr;
        v.x += o.x;
        v.y += o.y;
      }
      *gptr = v;
    }
  }
}

// A wave takes whole cells, a.cells_per_block / 4 of them one after the other, independently of the other waves of its
// block (they only share the block's LDS allocation): it stages x and y of a cell in its own piece of LDS, goes through
// the cell's runs, parks the two gradients in LDS and writes them out in whole rows.  One kernel per triple: each gets
// the registers its own body needs (one kernel with a switch over the triples spills in the larger bodies, since what
// is live around the switch comes on top of every body).
template <int L1, int L2, int D, bool WX, bool WY, int K>
__global__ void __launch_bounds__(kBlock)
    __attribute__((amdgpu_waves_per_eu(one_triple_small(L1, L2, cabs_(L1 - L2) + D, K) ? 4 : 1)))
one_triple_bwd_kernel(const BwdArgs a) {
  extern __shared__ float lds[];
  const int xsize = a.xsize, ysize = a.ysize, cpb = a.cells_per_block;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & (kWave - 1);
  float2 *xs = reinterpret_cast<float2 *>(lds) + wave * 2 * (xsize + ysize);
  float2 *ys = xs + xsize;
  float2 *ximg = ys + ysize;
  float2 *yimg = ximg + xsize;
  const PairPtr p = (PairPtr)a.pairs;
  const int per_wave = cpb / kWaves;
  const long long first = (long long)blockIdx.x * cpb + (long long)wave * per_wave;
  for (int t = 0; t < per_wave; t++) {
    const long long cell = first + t;
    if (cell >= a.ncells) break;
    if (WY) wave_copy_part<true>(a.x[0], a.xrows[0], xs, cell, lane, false);
    if (WX) wave_copy_part<true>(a.y[0], a.yrows[0], ys, cell, lane, false);
    __builtin_amdgcn_wave_barrier();
    one_triple_cell<L1, L2, D, WX, WY, K>(a, p, xs, ys, ximg, yimg, cell, lane);
    __builtin_amdgcn_wave_barrier();
    if (WX) wave_copy_part<false>(a.xg[0], a.xrows[0], ximg, cell, lane, a.accumulate != 0);
    if (WY) wave_copy_part<false>(a.yg[0], a.yrows[0], yimg, cell, lane, a.accumulate != 0);
    __builtin_amdgcn_wave_barrier();
  }
}

template <int N, int I = 0, typename F>
void host_for(F &&f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    host_for<N, I + 1>(f);
  }
}

// Launches the kernel of (l1, l2, l) if it belongs to the class SMALL of this translation unit.
template <int K, bool SMALL>
int launch_one_triple_k(const BwdArgs &a, int l1, int l2, int l, int nblocks, size_t lds, hipStream_t s) {
  const bool wx = a.want_x != 0, wy = a.want_y != 0;
  bool found = false;
  host_for<kLT + 1>([&](auto ac) {
    host_for<kLT + 1>([&](auto bc) {
      constexpr int A = decltype(ac)::value, B = decltype(bc)::value;
      host_for<2 * cmin_(A, B) + 1>([&](auto dc) {
        constexpr int D = decltype(dc)::value;
        if constexpr (one_triple_small(A, B, cabs_(A - B) + D, K) == SMALL) {
          if (l1 != A || l2 != B || l != cabs_(A - B) + D) return;
          found = true;
          if (wx && wy) hipLaunchKernelGGL((one_triple_bwd_kernel<A, B, D, true, true, K>), dim3(nblocks), dim3(kBlock), lds, s, a);
          else if (wx) hipLaunchKernelGGL((one_triple_bwd_kernel<A, B, D, true, false, K>), dim3(nblocks), dim3(kBlock), lds, s, a);
          else hipLaunchKernelGGL((one_triple_bwd_kernel<A, B, D, false, true, K>), dim3(nblocks), dim3(kBlock), lds, s, a);
        }
      });
    });
  });
  if (!found) return GELIB_HIP_ERR_UNSUPPORTED;
  GELIB_HIP_TRY(hipGetLastError());
  return GELIB_HIP_OK;
}

}  // namespace

}  // namespace gelib_hip
