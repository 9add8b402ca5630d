// Host side and helper kernels of the fused SO3vec CGproduct -> channel mixing forward pass (the kernel itself:
// cg_linear_impl.h): the matrices re-packed for the matrix cores, the first operand transposed per group of cells, the
// two launches.
#include <cstring>
#include <vector>

#include "cg_linear_impl.h"

namespace gelib_hip {

namespace {

// xt[group][e][slot] = x[cell 32 group + slot][e], e = row * n + channel; cells beyond the last repeat it.
__global__ void __launch_bounds__(256) transpose_cells_kernel(float2 *xt, const FastPart X, int elems, long long ncells) {
  __shared__ float2 tile[32][33];
  const long long g = blockIdx.x;
  const int e0 = blockIdx.y * 32, tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  for (int c = ty; c < 32; c += 8) {
    long long cell = g * 32 + c;
    cell = cell < ncells ? cell : ncells - 1;
    const int e = e0 + tx;
    if (e < elems) tile[c][tx] = X.ptr[cell * X.sb + (long long)(e / X.n) * X.sm + (e % X.n)];
  }
  __syncthreads();
  for (int ee = ty; ee < 32; ee += 8) {
    const int e = e0 + ee;
    if (e < elems) xt[(g * elems + e) * 32 + tx] = tile[tx][ee];
  }
}

// wp[c][h][2 o + p]: the real 2 x 2 form of W[c, o] = wr + i wi, rows h = (real, imaginary) part of the product's
// element, columns p = (real, imaginary) part of the result: [[wr, wi], [-wi, wr]]; columns beyond n_out are zero.
__global__ void pack_linear_kernel(float *wp, const float2 *w, long long tau, int n_out) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (tau + kBAhead) * 64) return;
  const long long c = idx >> 6;
  const int hh = (idx >> 5) & 1, col = idx & 31, o = col >> 1, p = col & 1;
  float val = 0.f;
  if (c < tau && o < n_out) {
    const float2 e = w[c * n_out + o];
    val = hh == 0 ? (p ? e.y : e.x) : (p ? e.x : -e.y);
  }
  wp[idx] = val;
}

size_t packed_bytes(long long tau) { return (size_t)(tau + kBAhead) * 256; }  // padding behind the last channel

}  // namespace

size_t cg_linear_workspace_bytes(const long long tau[kLinL + 1], long long x_elems_per_cell, long long ncells) {
  size_t total = 0;
  for (int l = 0; l <= kLinL; l++) total += packed_bytes(tau[l]);
  const long long groups = (ncells + kLinCells - 1) / kLinCells;
  return total + (size_t)groups * kLinCells * (size_t)x_elems_per_cell * sizeof(float2);
}

int cg_linear_fwd(const VecPlan &plan, const std::vector<const gelib_part_desc *> &r,
                  const std::vector<const gelib_part_desc *> &x, const std::vector<const gelib_part_desc *> &y,
                  const std::vector<const float2 *> &w, bool accumulate, void *ws, size_t ws_bytes, hipStream_t s,
                  int *used) {
  *used = 0;
  if (plan.diag) return GELIB_HIP_OK;
  std::vector<FastPart> fx, fy, fr;
  std::vector<std::pair<int, int>> lx, ly, lr;
  if (!lists_to_fast(x, plan.E, false, &fx, &lx) || !lists_to_fast(y, plan.E, false, &fy, &ly) ||
      !lists_to_fast(r, plan.E, true, &fr, &lr))
    return GELIB_HIP_OK;
  // every product part l = 0..kLinL, operands up to kLinL, narrow channels
  if ((int)lr.size() != kNL) return GELIB_HIP_OK;
  for (int l = 0; l < kNL; l++)
    if (lr[l].first != l || lr[l].second < 1 || lr[l].second > kLinMaxOut) return GELIB_HIP_OK;
  for (auto &p : lx)
    if (p.first > kLinL || p.second < 1 || p.second > kLinMaxN) return GELIB_HIP_OK;
  for (auto &p : ly)
    if (p.first > kLinL || p.second < 1 || p.second > kLinMaxN) return GELIB_HIP_OK;
  const long long ncells = plan.E[0] * plan.E[1] * plan.E[2];
  const long long nblocks = (ncells + kLinCells - 1) / kLinCells;
  if (nblocks > 0x7fffffffLL) return GELIB_HIP_OK;

  LinArgs a;
  std::memset(&a, 0, sizeof(a));
  for (size_t i = 0; i < fx.size(); i++) a.x[lx[i].first] = fx[i];
  for (size_t i = 0; i < fy.size(); i++) a.y[ly[i].first] = fy[i];
  for (int l = 0; l < kNL; l++) a.out[l] = fr[l];
  long long tau[kNL] = {0, 0, 0, 0, 0};
  for (auto &t : plan.triples) {
    a.offs[t.l1][t.l2][t.l] = t.offs;
    tau[t.l] = std::max(tau[t.l], (long long)t.offs + t.nout);
  }
  // a pair reaches every l of its range (every product part is there): the kernel relies on it
  for (auto &p : lx)
    for (auto &q : ly) {
      int have = 0;
      for (auto &t : plan.triples) have += (t.l1 == p.first && t.l2 == q.first);
      if (have != std::min(p.first + q.first, kLinL) - std::abs(p.first - q.first) + 1) return GELIB_HIP_OK;
    }
  long long x_elems = 0;
  for (auto &p : lx) x_elems += (long long)(2 * p.first + 1) * p.second;
  if (!ws || ((uintptr_t)ws & 15) || ws_bytes < cg_linear_workspace_bytes(tau, x_elems, ncells)) return GELIB_HIP_ERR_WORKSPACE;
  int rc = cg_table_bank(&a.bank);
  if (rc) return rc;
  a.ncells = ncells;
  a.accumulate = accumulate ? 1 : 0;
  char *cursor = (char *)ws;
  for (int l = 0; l < kNL; l++) {
    a.wp[l] = (const float *)cursor;
    const long long n = (tau[l] + kBAhead) * 64;
    pack_linear_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s>>>((float *)cursor, w[l], tau[l], lr[l].second);
    GELIB_HIP_TRY(hipGetLastError());
    cursor += packed_bytes(tau[l]);
  }
  for (size_t i = 0; i < fx.size(); i++) {
    const int l = lx[i].first, elems = (2 * l + 1) * lx[i].second;
    a.xt[l] = (const float2 *)cursor;
    transpose_cells_kernel<<<dim3((unsigned)nblocks, (unsigned)((elems + 31) / 32)), dim3(256), 0, s>>>((float2 *)cursor, fx[i], elems, ncells);
    GELIB_HIP_TRY(hipGetLastError());
    cursor += (size_t)nblocks * kLinCells * elems * sizeof(float2);
  }
  if ((rc = launch_cg_linear_pass0(a, nblocks, s))) return rc;
  if ((rc = launch_cg_linear_pass1(a, nblocks, s))) return rc;
  *used = 1;
  return GELIB_HIP_OK;
}

}  // namespace gelib_hip
