// Sum of slices along one leading dimension of a part:  r[.., t, ..] (+)= sum over the sources s of target t of
// x[.., s, ..]  -- the message-passing step that feeds the products (core/Gpart.hpp:537-563; the loop itself is
// cnine::GatherSlices, which is not part of the reference tree).
//
// The map arrives target-major (row_ptr / sources), so every output element is written by exactly one thread, which
// adds its sources in the order of the map: no atomics, and the float sum is reproducible.  Threads run along
// (target, other leading cells, m, channel) with the channel fastest, so the loads of one source slice and the store
// coalesce, and short slices do not leave lanes idle.
// HBM-bound: 8 B per (pair, element) read, 8 B per output element written (and read when accumulating).
#include <algorithm>

#include "cg_common.h"

namespace gelib_hip {

namespace {

struct GatherArgs {
  float2 *r;
  const float2 *x;
  long long rs[5], xs[5];  // strides in complex elements over (batch, grid0, grid1, m, channel)
  long long D[5];          // extents of r
  const int *row_ptr;      // [D[dim] + 1]
  const int *sources;      // [row_ptr[D[dim]]], each below the extent of x along dim
  int dim, accumulate;
};

__global__ void __launch_bounds__(256) gather_kernel(const GatherArgs a) {
  // extents with the gathered dimension taken out: one thread per element of a target slice, the element index
  // running fastest, so a wave covers 64 consecutive elements of one target (or the end of one and the start of the next)
  long long E[5];
  for (int k = 0; k < 5; k++) E[k] = k == a.dim ? 1 : a.D[k];
  const long long per_target = E[0] * E[1] * E[2] * E[3] * E[4];
  const long long total = per_target * a.D[a.dim];
  for (long long w = (long long)blockIdx.x * blockDim.x + threadIdx.x; w < total; w += (long long)gridDim.x * blockDim.x) {
    const long long t = w / per_target;
    long long rem = w - t * per_target, ro = t * a.rs[a.dim], xo = 0;
    for (int k = 4; k >= 0; k--) {
      const long long i = rem % E[k];
      rem /= E[k];
      ro += k == a.dim ? 0 : i * a.rs[k];
      xo += i * a.xs[k];   // i = 0 along the gathered dimension
    }
    float2 acc = a.accumulate ? a.r[ro] : make_float2(0.f, 0.f);
    const int k0 = a.row_ptr[t], k1 = a.row_ptr[t + 1];
    for (int k = k0; k < k1; k++) {
      const float2 v = a.x[xo + (long long)a.sources[k] * a.xs[a.dim]];
      acc.x += v.x;
      acc.y += v.y;
    }
    a.r[ro] = acc;
  }
}

}  // namespace

int launch_gather(float2 *r, const float2 *x, const long long rs[5], const long long xs[5], const long long D[5],
                  int dim, const int *row_ptr, const int *sources, bool accumulate, hipStream_t s) {
  GatherArgs a;
  a.r = r;
  a.x = x;
  long long per_target = 1;
  for (int k = 0; k < 5; k++) {
    a.rs[k] = rs[k];
    a.xs[k] = xs[k];
    a.D[k] = D[k];
    if (k != dim) per_target *= D[k];
  }
  a.dim = dim;
  a.row_ptr = row_ptr;
  a.sources = sources;
  a.accumulate = accumulate ? 1 : 0;
  if (per_target == 0 || D[dim] == 0) return 0;
  const long long total = per_target * D[dim];
  const long long want = (total + 255) / 256;
  hipLaunchKernelGGL(gather_kernel, dim3((unsigned)std::min<long long>(want, 256LL * 64)), dim3(256), 0, s, a);
  return hipGetLastError() == hipSuccess ? 0 : 10;
}

}  // namespace gelib_hip
