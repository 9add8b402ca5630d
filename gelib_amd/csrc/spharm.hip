// Spherical harmonics of 3-vectors into an SO3part: r[cell, L+m, j] (+)= Y_L^m(x[cell, :, j] / |x[cell, :, j]|).
//
// Same arithmetic as the reference's CPU loop (SO3/SO3part.hpp:340-403; CUDA twin cuda/SPharm.cu:30-85): the
// associated Legendre values are floats, each obtained from a double expression; the azimuthal phase runs as a
// complex float recurrence.  The reference fills a triangular table P(l,m), l <= L, and uses its last row; here a
// thread climbs l for one m at a time with the same three recurrences, so it needs two running values instead of a
// table in shared memory (which is what limits the reference to n*(L+1)(L+2)/2 floats of LDS per block).
// One thread per (cell, channel); channels are the fastest index of both tensors, so loads and stores coalesce.
// HBM-bound: 12 B read and (2L+1)*8 B written per thread.
#include <algorithm>

#include "cg_common.h"

// The recurrences amplify rounding differences, so multiply-adds are not fused here: every product and sum rounds as
// in the reference's host code.
#pragma clang fp contract(off)

namespace gelib_hip {

namespace {

struct SpharmArgs {
  PartDev r;
  const float *x;
  long long xsb, xsg0, xsg1, xsm, xsc;  // strides of x in floats (0 = broadcast)
  long long D[3];                        // cells
  int L, n, accumulate;
};

__global__ void __launch_bounds__(256) spharm_kernel(const SpharmArgs a) {
  const long long total = a.D[0] * a.D[1] * a.D[2] * a.n;
  const int L = a.L;
  const float norm = (float)sqrt((2.0 * L + 1.0) / (M_PI * 4.0));
  for (long long w = (long long)blockIdx.x * blockDim.x + threadIdx.x; w < total; w += (long long)gridDim.x * blockDim.x) {
    const long long cell = w / a.n;
    const int j = (int)(w - cell * a.n);
    const long long c2 = cell % a.D[2];
    const long long c1 = (cell / a.D[2]) % a.D[1];
    const long long c0 = cell / (a.D[2] * a.D[1]);
    const float *xp = a.x + c0 * a.xsb + c1 * a.xsg0 + c2 * a.xsg1 + (long long)j * a.xsc;
    float2 *rp = a.r.ptr + c0 * a.r.sb + c1 * a.r.sg0 + c2 * a.r.sg1 + (long long)j * a.r.sc;
    const float vx = xp[0], vy = xp[a.xsm], vz = xp[2 * a.xsm];
    const float length = sqrtf(vx * vx + vy * vy + vz * vz);
    const float len2 = sqrtf(vx * vx + vy * vy);
    auto put = [&](int row, float re, float im) {
      float2 *dst = rp + (long long)row * a.r.sm;
      float2 o = make_float2(re, im);
      if (a.accumulate) {
        const float2 old = *dst;
        o.x += old.x;
        o.y += old.y;
      }
      *dst = o;
    };
    if (len2 == 0 || isnan(vx / len2) || isnan(vy / len2)) {
      // a vector on the polar axis: only m = 0 (SO3/SO3part.hpp:364-366)
      if (a.accumulate) {
        put(L, (float)sqrt(((float)(2 * L + 1)) / (M_PI * 4.0)), 0.f);
      } else {
        for (int row = 0; row <= 2 * L; row++) put(row, row == L ? (float)sqrt(((float)(2 * L + 1)) / (M_PI * 4.0)) : 0.f, 0.f);
      }
      continue;
    }
    const float x = vz / length;
    const float xfact = (float)sqrt(1.0 - x * x);
    const float cr = vx / len2, ci = vy / len2;
    float pr = norm, pi = 0.f;
    float pmm = 1.f;  // P(m,m)
    for (int m = 0; m <= L; m++) {
      if (m > 0) pmm = (float)(-(2.0 * m - 1.0) * xfact * pmm);
      // climb l = m .. L at fixed m: P(m+1,m) = (2m+1) P(m,m) x, then the three-term recurrence
      float p2 = 0.f, p1 = pmm;  // P(l-2,m), P(l-1,m)
      if (m < L) {
        float cur = (float)((2.0 * (m + 1) - 1.0) * pmm * x);
        p2 = p1;
        p1 = cur;
        for (int l = m + 2; l <= L; l++) {
          cur = (float)(((2.0 * l - 1.0) * p1 * x - ((float)(l + m - 1.0)) * p2) / ((float)(l - m)));
          p2 = p1;
          p1 = cur;
        }
      }
      const float ar = pr * p1, ai = pi * p1;
      put(L + m, ar, ai);
      if (m > 0) {
        const float sg = (float)(1 - 2 * (m % 2));
        put(L - m, sg * ar, sg * (-ai));
      }
      if (m < L) {
        const float d = sqrtf((float)(L - m) * (L + m + 1));
        const float qr = cr / d, qi = ci / d;
        const float nr = pr * qr - pi * qi, ni = pr * qi + pi * qr;
        pr = nr;
        pi = ni;
      }
    }
  }
}

}  // namespace

int launch_spharm(const PartDev &r, const float *x, const long long xs[5], const long long D[3], int L, int n,
                  bool accumulate, hipStream_t s) {
  SpharmArgs a;
  a.r = r;
  a.x = x;
  a.xsb = xs[0], a.xsg0 = xs[1], a.xsg1 = xs[2], a.xsm = xs[3], a.xsc = xs[4];
  for (int k = 0; k < 3; k++) a.D[k] = D[k];
  a.L = L;
  a.n = n;
  a.accumulate = accumulate ? 1 : 0;
  const long long total = D[0] * D[1] * D[2] * n;
  if (total == 0) return GELIB_HIP_OK;
  const long long blocks = std::min<long long>((total + 255) / 256, 1 << 20);
  hipLaunchKernelGGL(spharm_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a);
  GELIB_HIP_TRY(hipGetLastError());
  return GELIB_HIP_OK;
}

}  // namespace gelib_hip
