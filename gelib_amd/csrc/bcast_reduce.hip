// Sum of per-cell gradients over the leading dimensions along which their destination broadcasts.
//
// A gradient destination with extent 1 where the operation has extent E (an operand shared by the whole batch or by the
// whole grid) is the sum of the per-cell gradients over that dimension (core/Gpart.hpp:168-185 makes such an operand a
// stride-0 view, and the reference's serial loops add every cell into the same memory).  The product kernels write one
// gradient per cell into a packed temporary; the kernels here add those up in two stages with a fixed order of
// additions (ranges of cells per thread, then the ranges in ascending order): no atomics, same bits every run.
#include <algorithm>

#include "cg_common.h"

namespace gelib_hip {

namespace {

struct ReduceArgs {
  const float2 *tmp;   // (E0, E1, E2, elems) packed
  float2 *part;        // partial sums (dcells, P, elems) when P > 1
  PartDev d;           // destination
  int E[3];            // extents of the temporary
  int D[3];            // extents of the destination (E[k] or 1)
  int n, elems;        // channels, (2l+1) * channels
  int Rn, P, len;      // cells summed per destination cell; ranges per destination cell; cells per range
  int accumulate;
};

// Coordinates of the summed cells of one destination cell: the dimensions along which the destination broadcasts run
// from 0 to E[k] - 1 (dimension 0 slowest), the others stay at the destination cell's own coordinate.
struct SummedCell {
  int c[3];   // coordinates in the temporary
  int R[3];   // extent of the summed range per dimension (1 where the destination has the dimension itself)
};

__device__ __forceinline__ SummedCell summed_cell(const ReduceArgs &a, int dc, int r) {
  SummedCell q;
  const int d2 = dc % a.D[2], d1 = (dc / a.D[2]) % a.D[1], d0 = dc / (a.D[2] * a.D[1]);
  q.R[0] = a.D[0] == 1 ? a.E[0] : 1, q.R[1] = a.D[1] == 1 ? a.E[1] : 1, q.R[2] = a.D[2] == 1 ? a.E[2] : 1;
  const int r2 = r % q.R[2], r1 = (r / q.R[2]) % q.R[1], r0 = r / (q.R[2] * q.R[1]);
  q.c[0] = a.D[0] == 1 ? r0 : d0, q.c[1] = a.D[1] == 1 ? r1 : d1, q.c[2] = a.D[2] == 1 ? r2 : d2;
  return q;
}
__device__ __forceinline__ long long cell_index(const ReduceArgs &a, const SummedCell &q) {
  return ((long long)q.c[0] * a.E[1] + q.c[1]) * a.E[2] + q.c[2];
}
// the next summed cell: the last summed dimension runs fastest
__device__ __forceinline__ void next_cell(const ReduceArgs &a, SummedCell &q) {
  if (q.R[2] > 1 && ++q.c[2] < a.E[2]) return;
  if (q.R[2] > 1) q.c[2] = 0;
  if (q.R[1] > 1 && ++q.c[1] < a.E[1]) return;
  if (q.R[1] > 1) q.c[1] = 0;
  if (q.R[0] > 1) ++q.c[0];
}

__device__ __forceinline__ float2 *dest_elem(const ReduceArgs &a, int dc, int e) {
  const int d2 = dc % a.D[2], d1 = (dc / a.D[2]) % a.D[1], d0 = dc / (a.D[2] * a.D[1]);
  const int row = e / a.n, ch = e - row * a.n;
  return a.d.ptr + d0 * a.d.sb + d1 * a.d.sg0 + d2 * a.d.sg1 + row * a.d.sm + ch * a.d.sc;
}

// thread = (destination cell, range, element), element fastest: the reads of a wave are contiguous
__global__ void __launch_bounds__(256) bcast_stage1_kernel(ReduceArgs a, long long total) {
  for (long long w = (long long)blockIdx.x * blockDim.x + threadIdx.x; w < total; w += (long long)gridDim.x * blockDim.x) {
    const int e = (int)(w % a.elems);
    const long long q = w / a.elems;
    const int p = (int)(q % a.P), dc = (int)(q / a.P);
    const int r0 = p * a.len, r1 = min(a.Rn, r0 + a.len);
    // eight loads in flight at a time (a thread's loads would otherwise wait for each other); the order of the additions
    // stays the order of the cells
    float2 acc = make_float2(0.f, 0.f);
    SummedCell sc = summed_cell(a, dc, r0);
    for (int r = r0; r < r1; r += 8) {
      float2 v[8];
#pragma unroll
      for (int u = 0; u < 8; u++) {
        v[u] = r + u < r1 ? a.tmp[cell_index(a, sc) * a.elems + e] : make_float2(0.f, 0.f);
        if (r + u < r1) next_cell(a, sc);
      }
#pragma unroll
      for (int u = 0; u < 8; u++) {
        acc.x += v[u].x;
        acc.y += v[u].y;
      }
    }
    if (a.P > 1) {
      a.part[w] = acc;
    } else {
      float2 *dst = dest_elem(a, dc, e);
      if (a.accumulate) {
        const float2 o = *dst;
        acc.x += o.x;
        acc.y += o.y;
      }
      *dst = acc;
    }
  }
}

__global__ void __launch_bounds__(256) bcast_stage2_kernel(ReduceArgs a, long long total) {
  for (long long w = (long long)blockIdx.x * blockDim.x + threadIdx.x; w < total; w += (long long)gridDim.x * blockDim.x) {
    const int e = (int)(w % a.elems), dc = (int)(w / a.elems);
    float2 acc = make_float2(0.f, 0.f);
    const float2 *pp = a.part + (long long)dc * a.P * a.elems + e;
    for (int p = 0; p < a.P; p += 8) {
      float2 v[8];
#pragma unroll
      for (int u = 0; u < 8; u++) v[u] = p + u < a.P ? pp[(long long)(p + u) * a.elems] : make_float2(0.f, 0.f);
#pragma unroll
      for (int u = 0; u < 8; u++) {
        acc.x += v[u].x;
        acc.y += v[u].y;
      }
    }
    float2 *dst = dest_elem(a, dc, e);
    if (a.accumulate) {
      const float2 o = *dst;
      acc.x += o.x;
      acc.y += o.y;
    }
    *dst = acc;
  }
}

// ranges per destination cell: enough threads to fill the GPU, at least 64 cells per range, and about as many ranges as
// cells per range (a thread of the second stage adds the ranges one after the other, as one of the first adds cells)
int choose_ranges(long long dcells, int elems, int Rn) {
  const long long want_threads = 1 << 18;
  long long P = want_threads / std::max<long long>(1, dcells * elems);
  P = std::min<long long>(P, Rn / 64);
  long long balanced = 1;
  while (balanced * balanced < Rn) balanced *= 2;
  P = std::min<long long>(P, balanced);
  return (int)std::max<long long>(1, P);
}

// dst[i] (+)= src[i]
__global__ void __launch_bounds__(256) add_into_kernel(float2 *dst, const float2 *src, long long n, int accumulate) {
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
    float2 v = src[i];
    if (accumulate) {
      const float2 o = dst[i];
      v.x += o.x;
      v.y += o.y;
    }
    dst[i] = v;
  }
}

}  // namespace

int launch_add_into(float2 *dst, const float2 *src, long long n, bool accumulate, hipStream_t s) {
  if (n <= 0) return GELIB_HIP_OK;
  hipLaunchKernelGGL(add_into_kernel, dim3((unsigned)std::min<long long>((n + 255) / 256, 1 << 16)), dim3(256), 0, s, dst, src,
                     n, accumulate ? 1 : 0);
  GELIB_HIP_TRY(hipGetLastError());
  return GELIB_HIP_OK;
}

size_t bcast_partial_bytes(const long long E[3], const long long D[3], int rows, int n) {
  long long dcells = D[0] * D[1] * D[2], Rn = 1;
  for (int k = 0; k < 3; k++)
    if (D[k] == 1) Rn *= E[k];
  const int P = choose_ranges(dcells, rows * n, (int)std::min<long long>(Rn, 0x7fffffff));
  return P > 1 ? (size_t)dcells * P * rows * n * sizeof(float2) : 0;
}

// tmp: packed (E0, E1, E2, rows, n); d: destination with own extents D (E[k] or 1); partial: bcast_partial_bytes() bytes
int launch_bcast_reduce(const float2 *tmp, float2 *partial, const PartDev &d, const long long E[3], const long long D[3],
                        int rows, int n, bool accumulate, hipStream_t s) {
  const long long cells = E[0] * E[1] * E[2], dcells = D[0] * D[1] * D[2];
  if (cells == 0 || rows * n == 0) return GELIB_HIP_OK;
  if (cells > 0x7fffffffLL || (long long)rows * n > 0x7fffffffLL) return GELIB_HIP_ERR_ARG;
  ReduceArgs a;
  a.tmp = tmp;
  a.part = partial;
  a.d = d;
  long long Rn = 1;
  for (int k = 0; k < 3; k++) {
    a.E[k] = (int)E[k];
    a.D[k] = (int)D[k];
    if (D[k] == 1) Rn *= E[k];
  }
  a.n = n;
  a.elems = rows * n;
  a.Rn = (int)Rn;
  a.P = choose_ranges(dcells, a.elems, a.Rn);
  a.len = (a.Rn + a.P - 1) / a.P;
  a.P = (a.Rn + a.len - 1) / a.len;   // no empty ranges
  a.accumulate = accumulate ? 1 : 0;
  if (a.P > 1 && !partial) return GELIB_HIP_ERR_WORKSPACE;
  const long long total1 = dcells * a.P * a.elems;
  auto grid = [](long long t) { return (unsigned)std::min<long long>((t + 255) / 256, 1 << 16); };
  hipLaunchKernelGGL(bcast_stage1_kernel, dim3(grid(total1)), dim3(256), 0, s, a, total1);
  GELIB_HIP_TRY(hipGetLastError());
  if (a.P > 1) {
    const long long total2 = dcells * a.elems;
    hipLaunchKernelGGL(bcast_stage2_kernel, dim3(grid(total2)), dim3(256), 0, s, a, total2);
    GELIB_HIP_TRY(hipGetLastError());
  }
  return GELIB_HIP_OK;
}

}  // namespace gelib_hip
