// Second kernel of an unrolled backward launch that dealt the pairs of a cell to several blocks (launches with few
// cells): adds the partial images of every cell in the order of the blocks and writes the gradients.
#include "cg_unrolled_dev.h"

namespace gelib_hip {

namespace {

constexpr int kMaxSplit = 32;  // the host deals the pairs of a cell to at most this many blocks

// One thread per element of the packed per-cell image of a part list: all of the element's partial sums are requested
// before the first is used (the loads of a thread do not wait for each other), added in the order of the blocks that
// wrote them, and stored to the element's place in its part.
template <int MAXS>
__device__ __forceinline__ void sum_images(const FastPart (&parts)[kFastIn], const int (&rows)[kFastIn], int nparts,
                                           const float2 *part, int size, long long ncells, int nsplit, bool accumulate) {
  const long long total = ncells * size;
  const long long slice = total;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (long long)gridDim.x * blockDim.x) {
    float2 v[MAXS];
#pragma unroll
    for (int w = 0; w < MAXS; w++) v[w] = part[(w < nsplit ? w : 0) * slice + e];
    float2 t = v[0];
#pragma unroll
    for (int w = 1; w < MAXS; w++)
      if (w < nsplit) {
        t.x += v[w].x;
        t.y += v[w].y;
      }
    const long long cell = e / size;
    int r = (int)(e - cell * size);
    float2 *dst = nullptr;
    static_for<kFastIn>([&](auto kc) __attribute__((always_inline)) {
      constexpr int k = decltype(kc)::value;
      if (k < nparts && dst == nullptr) {
        const int per_cell = rows[k] * parts[k].n;
        if (r < per_cell) {
          const int m = r / parts[k].n;
          dst = parts[k].ptr + cell * parts[k].sb + (long long)m * parts[k].sm + (r - m * parts[k].n);
        } else {
          r -= per_cell;
        }
      }
    });
    if (accumulate) {
      const float2 o = *dst;
      t.x += o.x;
      t.y += o.y;
    }
    *dst = t;
  }
}

template <int MAXS>
__global__ void __launch_bounds__(kBlock) unrolled_bwd_sum_splits_kernel(const BwdArgs a) {
  if (a.want_x) sum_images<MAXS>(a.xg, a.xrows, a.nx, a.part_x, a.xsize, a.ncells, a.pair_split, a.accumulate != 0);
  if (a.want_y) sum_images<MAXS>(a.yg, a.yrows, a.ny, a.part_y, a.ysize, a.ncells, a.pair_split, a.accumulate != 0);
}

}  // namespace

int launch_unrolled_bwd_sum_splits(const BwdArgs &a, int nblocks, hipStream_t s) {
  (void)nblocks;
  const long long elems = a.ncells * (long long)(a.xsize > a.ysize ? a.xsize : a.ysize);
  if (elems <= 0) return GELIB_HIP_OK;
  const long long grid = (elems + kBlock - 1) / kBlock;
  const dim3 g((unsigned)(grid < 65536 ? grid : 65536)), b(kBlock);
  if (a.pair_split > kMaxSplit) return GELIB_HIP_ERR_ARG;
  if (a.pair_split <= 4) hipLaunchKernelGGL(unrolled_bwd_sum_splits_kernel<4>, g, b, 0, s, a);
  else if (a.pair_split <= 8) hipLaunchKernelGGL(unrolled_bwd_sum_splits_kernel<8>, g, b, 0, s, a);
  else if (a.pair_split <= 16) hipLaunchKernelGGL(unrolled_bwd_sum_splits_kernel<16>, g, b, 0, s, a);
  else hipLaunchKernelGGL(unrolled_bwd_sum_splits_kernel<kMaxSplit>, g, b, 0, s, a);
  GELIB_HIP_TRY(hipGetLastError());
  return GELIB_HIP_OK;
}

}  // namespace gelib_hip
