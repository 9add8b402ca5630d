// Lane-per-channel Diag kernels for operand parts up to l = 2 (product up to l = 4), and backward kernels for operand
// parts up to l = 4 (gradient parts up to l = 6, or l = 7, 8 by themselves): a WAVE, not a block, takes a cell and 64
// channels (or the channels of several cells) and all of its (l1, l2) pairs.  Such a cell is a few
// kilobytes: with a block of four waves per cell, the staging of y in LDS, its barrier and the exchange of the
// x-gradient partial sums between the waves cost more than the arithmetic, and the launch is hundreds of thousands of
// blocks.  Here the waves of a block are independent (no barrier): forward everything is in registers; backward the
// x-gradient of a part stays in registers over all l2 and the y-gradient adds into a wave-private image in LDS
// (9 or 25 rows).  Same order of additions on every run.  Measured (one process): L=1, 64 channels, 355113 cells forward
// 1.40 -> 0.62 ms, backward 2.29 -> 0.88 ms; L=2, 16 channels, 1M cells 2.38 -> 1.86 and 2.82 -> 2.29 ms; L=4, 64
// channels, 131072 cells backward 7.1 -> 6.7 ms (forward the block form wins there, 5.6 against 6.8 ms, and is kept).
#include "cg_diag6_impl.h"

namespace gelib_hip {

namespace {

template <int kSmallLop, int kSmallCap, bool PACKED>
__global__ void __launch_bounds__(256) diag6_small_fwd_kernel(const Diag6Args a) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const long long w = (long long)blockIdx.x * 4 + wave;
  if (w >= a.nwaves) return;  // uniform for the wave; the kernel has no barrier
  const WavePos q = wave_pos(a, w);
  static_for<kSmallLop + 1>([&](auto l1c) __attribute__((always_inline)) {
    constexpr int L1 = decltype(l1c)::value;
    if (a.x[L1].ptr != nullptr) {
      float2 xv[2 * L1 + 1];
      load_rows<L1, PACKED>(xv, a.x[L1], q, a.xbc != 0);
      static_for<kSmallLop + 1>([&](auto l2c) __attribute__((always_inline)) {
        constexpr int L2 = decltype(l2c)::value;
        if (a.y[L2].ptr != nullptr) {
          float2 yv[2 * L2 + 1];
          load_rows<L2, PACKED>(yv, a.y[L2], q, a.ybc != 0);
          fwd_pair<L1, L2, kSmallCap, PACKED>(a, xv, yv, q);
        }
      });
    }
  });
}

template <int kSmallLop, int kSmallCap, bool PACKED, int LLO = 0>
__global__ void __launch_bounds__(256) diag6_small_bwd_kernel(const Diag6Args a) {
  constexpr int kYRows = (kSmallLop + 1) * (kSmallLop + 1);
  __shared__ float2 yimg_all[4 * kYRows * 64];  // [wave][row][lane]
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const long long w = (long long)blockIdx.x * 4 + wave;
  if (w >= a.nwaves) return;  // uniform for the wave; the kernel has no barrier
  const WavePos q = wave_pos(a, w);
  const bool accumulate = a.accumulate != 0;
  const bool wx = a.want_x != 0, wy = a.want_y != 0;
  // the wave's own image: only this wave touches it, and a wave's LDS operations execute in order
  float2 *yimg = yimg_all + wave * kYRows * 64;
#pragma unroll
  for (int r = 0; r < kYRows; r++) yimg[r * 64 + lane] = make_float2(0.f, 0.f);
  static_for<kSmallLop + 1>([&](auto l1c) __attribute__((always_inline)) {
    constexpr int L1 = decltype(l1c)::value;
    if constexpr (L1 + kSmallLop < LLO) return;  // no pair of this l1 reaches an l the launch takes
    if (a.x[L1].ptr != nullptr) {
      float2 xv[2 * L1 + 1], ax[2 * L1 + 1];
      if (wy) {
        load_rows<L1, PACKED>(xv, a.x[L1], q, a.xbc != 0);
      } else {
#pragma unroll
        for (int m1 = 0; m1 <= 2 * L1; m1++) xv[m1] = make_float2(0.f, 0.f);
      }
#pragma unroll
      for (int m1 = 0; m1 <= 2 * L1; m1++) ax[m1] = make_float2(0.f, 0.f);
      static_for<kSmallLop + 1>([&](auto l2c) __attribute__((always_inline)) {
        constexpr int L2 = decltype(l2c)::value;
        if (a.y[L2].ptr != nullptr) {
          float2 yv[2 * L2 + 1];
          if (wx) {
            load_rows<L2, PACKED>(yv, a.y[L2], q, a.ybc != 0);
          } else {
#pragma unroll
            for (int m2 = 0; m2 <= 2 * L2; m2++) yv[m2] = make_float2(0.f, 0.f);
          }
          if constexpr (L1 + L2 >= LLO) bwd_pair<L1, L2, kSmallCap, PACKED, LLO>(a, xv, yv, ax, yimg, q);
        }
      });
      if (wx && a.xg[L1].ptr != nullptr) store_rows<L1, PACKED>(ax, 1, a.xg[L1], q, accumulate, a.xbc != 0, a.lg_npad);
    }
  });
  static_for<kSmallLop + 1>([&](auto l2c) __attribute__((always_inline)) {
    constexpr int L2 = decltype(l2c)::value;
    const FastPart YG = a.yg[L2];
    if constexpr (L2 + kSmallLop >= LLO) {
      if (wy && YG.ptr != nullptr)
        store_rows<L2, PACKED>(yimg + (L2 * L2) * 64 + lane, 64, YG, q, accumulate, a.ybc != 0, a.lg_npad);
    }
  });
}

template <int LOP, int LCAP, int LLO = 0>
int launch_small(bool bwd, const Diag6Args &a, hipStream_t s) {
  const unsigned nblocks = (unsigned)((a.nwaves + 3) / 4);
  if (bwd) {
    if (a.lg_npad < 6) hipLaunchKernelGGL((diag6_small_bwd_kernel<LOP, LCAP, true, LLO>), dim3(nblocks), dim3(256), 0, s, a);
    else hipLaunchKernelGGL((diag6_small_bwd_kernel<LOP, LCAP, false, LLO>), dim3(nblocks), dim3(256), 0, s, a);
  } else {
    if (a.lg_npad < 6) hipLaunchKernelGGL((diag6_small_fwd_kernel<LOP, LCAP, true>), dim3(nblocks), dim3(256), 0, s, a);
    else hipLaunchKernelGGL((diag6_small_fwd_kernel<LOP, LCAP, false>), dim3(nblocks), dim3(256), 0, s, a);
  }
  GELIB_HIP_TRY(hipGetLastError());
  return GELIB_HIP_OK;
}

}  // namespace

int launch_diag6_small_fwd(const Diag6Args &a, hipStream_t s) { return launch_small<2, 4>(false, a, s); }
int launch_diag6_small_bwd(const Diag6Args &a, hipStream_t s) { return launch_small<2, 4>(true, a, s); }
int launch_diag6_small4_bwd(const Diag6Args &a, hipStream_t s) { return launch_small<4, 6>(true, a, s); }
int launch_diag6_small4_hi_bwd(const Diag6Args &a, hipStream_t s) { return launch_small<4, 8, 7>(true, a, s); }

}  // namespace gelib_hip
