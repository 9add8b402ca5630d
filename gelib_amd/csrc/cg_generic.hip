// Shape-agnostic kernels: any l up to GELIB_HIP_MAX_L, any channel counts, any strides, broadcast operands and
// broadcast destinations (a destination with extent 1 where the operation has extent E is summed over that axis,
// as the reference's serial CPU loop does, core/Gpart.hpp:325-360).
//
// Common layout choices:
//   * the (2l1+1)x(2l2+1) coefficient table is staged in LDS once per block;
//   * adjacent lanes own adjacent channels of the widest tensor (the product r or its gradient g), so its
//     rows are read and written as contiguous runs when the channel stride is 1;
//   * 64-bit offsets for everything that scales with the batch.
#include "cg_common.h"

namespace gelib_hip {

namespace {

struct GenericArgs {
  PartDev r, x, y;
  long long D[3];   // extents of the destination (parallel cells)
  long long Rd[3];  // extents summed over inside a thread (E[d]/D[d], i.e. E[d] where the destination broadcasts)
  const float *C;   // device table (2l1+1)x(2l2+1)
  int l1, l2, l, n1, n2, offs;
  int accumulate;
};

__device__ __forceinline__ void stage_table(float *Cs, const float *C, int n) {
  for (int i = threadIdx.x; i < n; i += blockDim.x) Cs[i] = C[i];
  __syncthreads();
}

__device__ __forceinline__ float2 cmul(float2 a, float2 b) {
  return make_float2(a.x * b.x - a.y * b.y, a.x * b.y + a.y * b.x);
}
__device__ __forceinline__ float2 cmul_conj(float2 a, float2 b) {  // a * conj(b)
  return make_float2(a.x * b.x + a.y * b.y, a.y * b.x - a.x * b.y);
}

// offset of cell (c0+q0, c1+q1, c2+q2) where broadcast dimensions carry stride 0
__device__ __forceinline__ long long cell_off(const PartDev &p, long long c0, long long c1, long long c2) {
  return c0 * p.sb + c1 * p.sg0 + c2 * p.sg1;
}

// ---- forward: one thread per (destination cell, output channel) ------------------------------------------------
template <bool DIAG>
__global__ void __launch_bounds__(256) generic_fwd_kernel(GenericArgs a) {
  extern __shared__ float Cs[];
  const int L2 = 2 * a.l2 + 1;
  stage_table(Cs, a.C, (2 * a.l1 + 1) * L2);

  const long long U = DIAG ? a.n1 : (long long)a.n1 * a.n2;
  const long long cells = a.D[0] * a.D[1] * a.D[2];
  const long long total = cells * U;
  for (long long w = (long long)blockIdx.x * blockDim.x + threadIdx.x; w < total; w += (long long)gridDim.x * blockDim.x) {
    const long long cell = w / U;
    const int u = (int)(w - cell * U);
    const int i = DIAG ? u : u / a.n2;
    const int j = DIAG ? u : u - i * a.n2;
    const long long c2 = cell % a.D[2];
    const long long c1 = (cell / a.D[2]) % a.D[1];
    const long long c0 = cell / (a.D[2] * a.D[1]);
    float2 *rp = a.r.ptr + cell_off(a.r, c0, c1, c2) + (long long)(a.offs + u) * a.r.sc;
    for (int m = -a.l; m <= a.l; m++) {
      float2 acc = make_float2(0.f, 0.f);
      const int m1lo = max(-a.l1, m - a.l2), m1hi = min(a.l1, m + a.l2);
      for (long long q0 = 0; q0 < a.Rd[0]; q0++)
        for (long long q1 = 0; q1 < a.Rd[1]; q1++)
          for (long long q2 = 0; q2 < a.Rd[2]; q2++) {
            const float2 *xp = a.x.ptr + cell_off(a.x, c0 + q0, c1 + q1, c2 + q2) + (long long)i * a.x.sc;
            const float2 *yp = a.y.ptr + cell_off(a.y, c0 + q0, c1 + q1, c2 + q2) + (long long)j * a.y.sc;
            for (int m1 = m1lo; m1 <= m1hi; m1++) {
              const int m2 = m - m1;
              const float c = Cs[(m1 + a.l1) * L2 + (m2 + a.l2)];
              const float2 xv = xp[(m1 + a.l1) * a.x.sm];
              const float2 yv = yp[(m2 + a.l2) * a.y.sm];
              const float2 t = cmul(make_float2(c * xv.x, c * xv.y), yv);
              acc.x += t.x;
              acc.y += t.y;
            }
          }
      float2 *dst = rp + (long long)(m + a.l) * a.r.sm;
      if (a.accumulate) {
        const float2 o = *dst;
        acc.x += o.x;
        acc.y += o.y;
      }
      *dst = acc;
    }
  }
}

// ---- back0 (CG): destination xg[m1,i]; lanes run along the reduced channel j so g is read contiguously, then a
// shuffle reduction inside aligned groups of n2p lanes; several (cell,i) pairs share a wave when n2 is small. --------
__global__ void __launch_bounds__(256) generic_back0_kernel(GenericArgs a, int n2p) {
  extern __shared__ float Cs[];
  const int L2 = 2 * a.l2 + 1;
  stage_table(Cs, a.C, (2 * a.l1 + 1) * L2);

  const int groups_per_block = blockDim.x / n2p;
  const int grp = threadIdx.x / n2p;
  const int jl = threadIdx.x - grp * n2p;
  const long long cells = a.D[0] * a.D[1] * a.D[2];
  const long long items = cells * a.n1;  // (destination cell, i)
  // every lane of a wave runs the same number of iterations: the bound is per block
  for (long long base = (long long)blockIdx.x * groups_per_block; base < items; base += (long long)gridDim.x * groups_per_block) {
    const long long q = base + grp;
    const bool live = q < items;
    const long long cell = live ? q / a.n1 : 0;
    const int i = live ? (int)(q - cell * a.n1) : 0;
    const long long c2 = cell % a.D[2];
    const long long c1 = (cell / a.D[2]) % a.D[1];
    const long long c0 = cell / (a.D[2] * a.D[1]);
    float2 *xg = a.x.ptr + cell_off(a.x, c0, c1, c2) + (long long)i * a.x.sc;
    for (int m1 = -a.l1; m1 <= a.l1; m1++) {
      float2 acc = make_float2(0.f, 0.f);
      const int m2lo = max(-a.l2, -a.l - m1), m2hi = min(a.l2, a.l - m1);
      if (live) {
        for (long long q0 = 0; q0 < a.Rd[0]; q0++)
          for (long long q1 = 0; q1 < a.Rd[1]; q1++)
            for (long long q2 = 0; q2 < a.Rd[2]; q2++) {
              const float2 *gp = a.r.ptr + cell_off(a.r, c0 + q0, c1 + q1, c2 + q2);
              const float2 *yp = a.y.ptr + cell_off(a.y, c0 + q0, c1 + q1, c2 + q2);
              for (int j = jl; j < a.n2; j += n2p) {
                const long long gch = (long long)(a.offs + i * a.n2 + j) * a.r.sc;
                for (int m2 = m2lo; m2 <= m2hi; m2++) {
                  const float c = Cs[(m1 + a.l1) * L2 + (m2 + a.l2)];
                  const float2 gv = gp[(long long)(m1 + m2 + a.l) * a.r.sm + gch];
                  const float2 yv = yp[(long long)(m2 + a.l2) * a.y.sm + (long long)j * a.y.sc];
                  const float2 t = cmul_conj(make_float2(c * gv.x, c * gv.y), yv);
                  acc.x += t.x;
                  acc.y += t.y;
                }
              }
            }
      }
      for (int s = 1; s < n2p; s <<= 1) {
        acc.x += __shfl_xor(acc.x, s);
        acc.y += __shfl_xor(acc.y, s);
      }
      if (live && jl == 0) {
        float2 *dst = xg + (long long)(m1 + a.l1) * a.x.sm;
        if (a.accumulate) {
          const float2 o = *dst;
          acc.x += o.x;
          acc.y += o.y;
        }
        *dst = acc;
      }
    }
  }
}

// ---- serial-reduction backward: one thread per (destination cell, destination channel d).
// MODE 0: CG back1   dest yg[m2,j], partner x[m1,i], reduce over i in-thread (g read contiguously across lanes j)
// MODE 1: Diag back0 dest xg[m1,c], partner y[m2,c]
// MODE 2: Diag back1 dest yg[m2,c], partner x[m1,c]
template <int MODE>
__global__ void __launch_bounds__(256) generic_back_serial_kernel(GenericArgs a) {
  extern __shared__ float Cs[];
  const int L2 = 2 * a.l2 + 1;
  stage_table(Cs, a.C, (2 * a.l1 + 1) * L2);

  constexpr bool DEST_IS_X = (MODE == 1);
  const PartDev &dst_t = DEST_IS_X ? a.x : a.y;
  const PartDev &par_t = DEST_IS_X ? a.y : a.x;
  const int ld = DEST_IS_X ? a.l1 : a.l2;   // l of the destination
  const int lp = DEST_IS_X ? a.l2 : a.l1;   // l of the partner
  const int nd = DEST_IS_X ? a.n1 : a.n2;
  const int nred = (MODE == 0) ? a.n1 : 1;

  const long long cells = a.D[0] * a.D[1] * a.D[2];
  const long long total = cells * nd;
  for (long long w = (long long)blockIdx.x * blockDim.x + threadIdx.x; w < total; w += (long long)gridDim.x * blockDim.x) {
    const long long cell = w / nd;
    const int d = (int)(w - cell * nd);
    const long long c2 = cell % a.D[2];
    const long long c1 = (cell / a.D[2]) % a.D[1];
    const long long c0 = cell / (a.D[2] * a.D[1]);
    float2 *dp = dst_t.ptr + cell_off(dst_t, c0, c1, c2) + (long long)d * dst_t.sc;
    for (int md = -ld; md <= ld; md++) {
      float2 acc = make_float2(0.f, 0.f);
      const int mplo = max(-lp, -a.l - md), mphi = min(lp, a.l - md);
      for (long long q0 = 0; q0 < a.Rd[0]; q0++)
        for (long long q1 = 0; q1 < a.Rd[1]; q1++)
          for (long long q2 = 0; q2 < a.Rd[2]; q2++) {
            const float2 *gp = a.r.ptr + cell_off(a.r, c0 + q0, c1 + q1, c2 + q2);
            const float2 *pp = par_t.ptr + cell_off(par_t, c0 + q0, c1 + q1, c2 + q2);
            for (int e = 0; e < nred; e++) {
              const int pch = (MODE == 0) ? e : d;
              const long long gch = (long long)(a.offs + ((MODE == 0) ? e * a.n2 + d : d)) * a.r.sc;
              for (int mp = mplo; mp <= mphi; mp++) {
                const int m1 = DEST_IS_X ? md : mp;
                const int m2 = DEST_IS_X ? mp : md;
                const float c = Cs[(m1 + a.l1) * L2 + (m2 + a.l2)];
                const float2 gv = gp[(long long)(md + mp + a.l) * a.r.sm + gch];
                const float2 pv = pp[(long long)(mp + lp) * par_t.sm + (long long)pch * par_t.sc];
                const float2 t = cmul_conj(make_float2(c * gv.x, c * gv.y), pv);
                acc.x += t.x;
                acc.y += t.y;
              }
            }
          }
      float2 *dst = dp + (long long)(md + ld) * dst_t.sm;
      if (a.accumulate) {
        const float2 o = *dst;
        acc.x += o.x;
        acc.y += o.y;
      }
      *dst = acc;
    }
  }
}

__global__ void __launch_bounds__(256) zero_fill_kernel(PartDev d, long long D0, long long D1, long long D2, int M, int n) {
  const long long per_cell = (long long)M * n;
  const long long total = D0 * D1 * D2 * per_cell;
  for (long long w = (long long)blockIdx.x * blockDim.x + threadIdx.x; w < total; w += (long long)gridDim.x * blockDim.x) {
    const long long cell = w / per_cell;
    const int e = (int)(w - cell * per_cell);
    const int m = e / n, c = e - m * n;
    const long long c2 = cell % D2, c1 = (cell / D2) % D1, c0 = cell / (D2 * D1);
    d.ptr[cell_off(d, c0, c1, c2) + (long long)m * d.sm + (long long)c * d.sc] = make_float2(0.f, 0.f);
  }
}

int grid_for(long long total_threads) {
  long long blocks = (total_threads + 255) / 256;
  const long long cap = 256LL * 64;  // grid-stride beyond this
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return (int)blocks;
}

int fill_args(const PartOp &op, const long long Dest[3], bool accumulate, GenericArgs &a) {
  a.r = op.r;
  a.x = op.x;
  a.y = op.y;
  for (int d = 0; d < 3; d++) {
    a.D[d] = Dest[d];
    a.Rd[d] = (Dest[d] == op.E[d]) ? 1 : op.E[d];
  }
  a.l1 = op.l1;
  a.l2 = op.l2;
  a.l = op.l;
  a.n1 = op.n1;
  a.n2 = op.n2;
  a.offs = op.offs;
  a.accumulate = accumulate ? 1 : 0;
  return cg_matrix_device(op.l1, op.l2, op.l, &a.C);
}

}  // namespace

int launch_generic_fwd(const PartOp &op, bool accumulate, hipStream_t s) {
  GenericArgs a;
  int rc = fill_args(op, op.Dr, accumulate, a);
  if (rc) return rc;
  const long long cells = a.D[0] * a.D[1] * a.D[2];
  if (cells == 0 || op.nout == 0) return GELIB_HIP_OK;
  const size_t lds = sizeof(float) * (size_t)(2 * op.l1 + 1) * (2 * op.l2 + 1);
  const int grid = grid_for(cells * op.nout);
  if (op.diag)
    hipLaunchKernelGGL(generic_fwd_kernel<true>, dim3(grid), dim3(256), lds, s, a);
  else
    hipLaunchKernelGGL(generic_fwd_kernel<false>, dim3(grid), dim3(256), lds, s, a);
  GELIB_HIP_TRY(hipGetLastError());
  return GELIB_HIP_OK;
}

int launch_generic_back0(const PartOp &op, bool accumulate, hipStream_t s) {
  GenericArgs a;
  int rc = fill_args(op, op.Dx, accumulate, a);
  if (rc) return rc;
  const long long cells = a.D[0] * a.D[1] * a.D[2];
  if (cells == 0 || op.n1 == 0) return GELIB_HIP_OK;
  const size_t lds = sizeof(float) * (size_t)(2 * op.l1 + 1) * (2 * op.l2 + 1);
  if (op.diag) {
    hipLaunchKernelGGL(generic_back_serial_kernel<1>, dim3(grid_for(cells * op.n1)), dim3(256), lds, s, a);
  } else {
    int n2p = 1;
    while (n2p < op.n2 && n2p < kWave) n2p <<= 1;
    const long long items = cells * op.n1;
    const int groups_per_block = 256 / n2p;
    long long blocks = (items + groups_per_block - 1) / groups_per_block;
    if (blocks > 256LL * 64) blocks = 256LL * 64;
    hipLaunchKernelGGL(generic_back0_kernel, dim3((int)blocks), dim3(256), lds, s, a, n2p);
  }
  GELIB_HIP_TRY(hipGetLastError());
  return GELIB_HIP_OK;
}

int launch_generic_back1(const PartOp &op, bool accumulate, hipStream_t s) {
  GenericArgs a;
  int rc = fill_args(op, op.Dy, accumulate, a);
  if (rc) return rc;
  const long long cells = a.D[0] * a.D[1] * a.D[2];
  if (cells == 0 || op.n2 == 0) return GELIB_HIP_OK;
  const size_t lds = sizeof(float) * (size_t)(2 * op.l1 + 1) * (2 * op.l2 + 1);
  const int grid = grid_for(cells * op.n2);
  if (op.diag)
    hipLaunchKernelGGL(generic_back_serial_kernel<2>, dim3(grid), dim3(256), lds, s, a);
  else
    hipLaunchKernelGGL(generic_back_serial_kernel<0>, dim3(grid), dim3(256), lds, s, a);
  GELIB_HIP_TRY(hipGetLastError());
  return GELIB_HIP_OK;
}

int launch_zero_fill(const PartDev &d, const long long D[3], int M, int n, hipStream_t s) {
  const long long total = D[0] * D[1] * D[2] * (long long)M * n;
  if (total == 0) return GELIB_HIP_OK;
  hipLaunchKernelGGL(zero_fill_kernel, dim3(grid_for(total)), dim3(256), 0, s, d, D[0], D[1], D[2], M, n);
  GELIB_HIP_TRY(hipGetLastError());
  return GELIB_HIP_OK;
}

}  // namespace gelib_hip
