// Backward pass of a product with ONE x part and ONE y part of any l (l1 + l2 <= 21, at most 21 values of l, at most
// 64 channel slots per cell), both gradients from one pass over g -- the "all l of one pair" case, e.g. l1 = l2 = 10.
//
// A wave takes 64 channel slots (one or more whole cells); a lane owns one channel pair (i, j) (Diag: one channel).
// The loops over m = m1 + m2 and over m1 run at run time, the loop over the l of the pair is unrolled: for one m the
// lane holds the rows g_l[m] of every l in registers (static indices), reads the coefficients C_l[m1, m - m1] of all l
// as one contiguous, zero-padded record through scalar loads, contracts over l first,
//     Q = sum_l C_l[m1, m2] g_l[m],
// and feeds both gradients once per (m1, m2): ax[m1] += Q conj(y[m2]), ay[m2] += Q conj(x[m1]).  The sums ax, ay live
// in LDS, one column per lane, so that the run-time row index costs an address, not a register-file lookup.  After
// the last m the columns are summed across the lanes that share i (resp. j) and written out.  No atomics, a fixed
// order of additions.
#include <cstring>
#include <map>
#include <mutex>
#include <vector>

#include "cg_lane_sums.h"
#include "cg_staged.h"
#include "cg_unrolled_dev.h"

namespace gelib_hip {

namespace {

constexpr int kNL = 21;      // most values of l one pair may have here
constexpr int kRecord = 24;  // floats per coefficient record (kNL rounded up, so that records stay 32-byte aligned)
constexpr int kMaxRows = 44; // (2 l1 + 1) + (2 l2 + 1) at most: the LDS columns of a wave
constexpr int kStepsMax = 22; // steps of one m (at most 21 when l1 + l2 <= 21) plus one that is read ahead: 64 lanes x 8
                              // floats = 512 floats cover 21 records, the 22nd slot stays whatever it was

struct OnePairArgs {
  FastPart x, y, xg, yg;
  FastPart g[kNL];    // by dl = l - lmin; ptr == nullptr: no such triple
  int offs[kNL];      // first channel of the triple's block in its part
  const float *coef;  // device: one record of kRecord floats per (m, m1) step, m ascending, then m1 ascending
  const int *mstart;  // device: number of the first step of every m, m = -lt .. lt
  long long ncells;
  int l1, l2, lmin, lt;  // lt = largest |m| that occurs
  int n1, n2;
  int log2_u, lg_n2p;    // lane slots per cell n1p * n2p (Diag: n1p) and n2p, as logs
  int diag;
  int offs_add, accumulate;
  int rec_off;  // float2 offset of the record buffers in LDS (16-byte aligned)
};

typedef float v2f __attribute__((ext_vector_type(2)));
typedef const __attribute__((address_space(1))) v2f *GlobalIn;
typedef __attribute__((address_space(1))) v2f *GlobalOut;
typedef const __attribute__((address_space(4))) float *CoeffPtr;
typedef const __attribute__((address_space(4))) int *IntPtr;

template <bool DIAG>
__global__ void __launch_bounds__(64) onepair_bwd_kernel(const OnePairArgs a) {
  extern __shared__ float2 lds[];
  const int lane = threadIdx.x;
  const int l1 = a.l1, l2 = a.l2, lmin = a.lmin, lt = a.lt, n1 = a.n1, n2 = a.n2;
  const int r1 = 2 * l1 + 1, r2 = 2 * l2 + 1;
  const int cpw = 64 >> a.log2_u;
  float2 *accx = lds;               // [r1][64]
  float2 *accy = accx + r1 * 64;    // [r2][64]
  float2 *xs = accy + r2 * 64;      // [cpw][r1][n1]
  float2 *ys = xs + cpw * r1 * n1;  // [cpw][r2][n2]
  float4 *recs = reinterpret_cast<float4 *>(lds + a.rec_off);  // [kStepsMax * kRecord / 4]: coefficient records of one m

  const long long cell0 = (long long)blockIdx.x * cpw;
  const int u = lane & ((1 << a.log2_u) - 1);
  int cell_local = lane >> a.log2_u;
  int i = DIAG ? u : (u >> a.lg_n2p);
  int j = DIAG ? u : (u & ((1 << a.lg_n2p) - 1));
  const bool valid = i < n1 && j < n2 && cell0 + cell_local < a.ncells;
  if (!valid) cell_local = 0, i = 0, j = 0;  // reads valid memory; its g is forced to zero and it never writes
  const int chan = DIAG ? i : i * n2 + j;

  for (int r = 0; r < r1 + r2; r++) accx[r * 64 + lane] = make_float2(0.f, 0.f);
  {
    const long long left = a.ncells - cell0;
    const int ncell = left < cpw ? (int)left : cpw;
    for (int e = lane; e < ncell * r1 * n1; e += 64) {
      const int c = e / (r1 * n1), rem = e - c * (r1 * n1), m = rem / n1, ch = rem - m * n1;
      xs[e] = a.x.ptr[(cell0 + c) * a.x.sb + (long long)m * a.x.sm + ch];
    }
    for (int e = lane; e < ncell * r2 * n2; e += 64) {
      const int c = e / (r2 * n2), rem = e - c * (r2 * n2), m = rem / n2, ch = rem - m * n2;
      ys[e] = a.y.ptr[(cell0 + c) * a.y.sb + (long long)m * a.y.sm + ch];
    }
  }
  __syncthreads();

  // per part: the address of the lane's element in the row that is read next (rows are read in ascending order, one
  // per m while |m| <= l), and the distance between rows
  typedef __attribute__((address_space(1))) char *LanePtr;
  LanePtr next_row[kNL];
  static_for<kNL>([&](auto dc) __attribute__((always_inline)) {
    constexpr int dl = decltype(dc)::value;
    const FastPart P = a.g[dl];
    const int L = lmin + dl;
    const int first = L > lt ? L - lt : 0;  // row m + L of the first m = -min(L, lt)
    next_row[dl] = (LanePtr)P.ptr + (((cell0 + cell_local) * P.sb + (long long)first * P.sm) + (a.offs[dl] + a.offs_add + chan)) * 8;
  });

  auto load_m = [&](int m, float2(&G)[kNL]) __attribute__((always_inline)) {
    const int mabs = m < 0 ? -m : m;
    static_for<kNL>([&](auto dc) __attribute__((always_inline)) {
      constexpr int dl = decltype(dc)::value;
      G[dl] = make_float2(0.f, 0.f);
      if (a.g[dl].ptr != nullptr && lmin + dl >= mabs) {  // uniform
        const v2f t = *(GlobalIn)next_row[dl];
        next_row[dl] += (long long)a.g[dl].sm * 8;
        if (valid) G[dl] = make_float2(t.x, t.y);
      }
    });
  };

  const IntPtr mstart = (IntPtr)a.mstart;
  const float2 *xcol = xs + cell_local * r1 * n1 + i;
  const float2 *ycol = ys + cell_local * r2 * n2 + j;
  // The records of one m (at most 21 steps of 24 floats) are fetched one m ahead, 8 floats per lane, and parked in
  // LDS; the inner loop then reads them as broadcasts with the latency of LDS.  (Scalar loads straight from the
  // table cost an L2 round trip per step once the table outgrows the scalar cache -- 42 KB for l1 = l2 = 10.)
  auto load_recs = [&](int m, float4(&R)[2]) __attribute__((always_inline)) {
    const float4 *src = reinterpret_cast<const float4 *>(a.coef + (long long)mstart[m + lt] * kRecord) + lane * 2;
    R[0] = src[0];  // the table ends with enough spare floats for the last m
    R[1] = src[1];
  };
  float2 Gn[kNL];
  float4 Rn[2];
  load_m(-lt, Gn);
  load_recs(-lt, Rn);
  for (int m = -lt; m <= lt; m++) {
    float2 G[kNL];
#pragma unroll
    for (int k = 0; k < kNL; k++) G[k] = Gn[k];
    float4 *buf = recs;  // one buffer: the wave's reads of the last m precede these writes in program order
    buf[lane * 2] = Rn[0];
    buf[lane * 2 + 1] = Rn[1];
    if (m < lt) {
      load_m(m + 1, Gn);
      load_recs(m + 1, Rn);
    }
    __syncthreads();  // one wave: makes the records written by the other lanes visible
    const int m1lo = max(-l1, m - l2), m1hi = min(l1, m + l2);
    float c[kRecord];
    auto read_rec = [&](int k, float(&dst)[kRecord]) __attribute__((always_inline)) {
#pragma unroll
      for (int q4 = 0; q4 < kRecord / 4; q4++) {
        const float4 t = buf[k * (kRecord / 4) + q4];
        dst[4 * q4] = t.x, dst[4 * q4 + 1] = t.y, dst[4 * q4 + 2] = t.z, dst[4 * q4 + 3] = t.w;
      }
    };
    // one step: the record of the next step is requested first (the buffer has room for one step beyond the last),
    // then this step's values from LDS; both arrive while the contraction over l runs
    auto step = [&](int m1, const float(&cc)[kRecord], float(&cnext)[kRecord]) __attribute__((always_inline)) {
      const int m2 = m - m1;
      read_rec(m1 - m1lo + 1, cnext);
      const float2 xc = xcol[(m1 + l1) * n1], yc = ycol[(m2 + l2) * n2];
      float2 *px = accx + (m1 + l1) * 64 + lane, *py = accy + (m2 + l2) * 64 + lane;
      float2 sx = *px, sy = *py;
      float qr = 0.f, qi = 0.f;
#pragma unroll
      for (int dl = 0; dl < kNL; dl++) {
        qr = fmaf(cc[dl], G[dl].x, qr);
        qi = fmaf(cc[dl], G[dl].y, qi);
      }
      sx.x = fmaf(qr, yc.x, sx.x);
      sx.x = fmaf(qi, yc.y, sx.x);
      sx.y = fmaf(qi, yc.x, sx.y);
      sx.y = fmaf(-qr, yc.y, sx.y);
      sy.x = fmaf(qr, xc.x, sy.x);
      sy.x = fmaf(qi, xc.y, sy.x);
      sy.y = fmaf(qi, xc.x, sy.y);
      sy.y = fmaf(-qr, xc.y, sy.y);
      *px = sx;
      *py = sy;
    };
    float cb[kRecord];
    read_rec(0, c);
    for (int m1 = m1lo; m1 <= m1hi; m1 += 2) {  // two steps per turn, so that the two record buffers swap by name
      step(m1, c, cb);
      if (m1 + 1 <= m1hi) step(m1 + 1, cb, c);
    }
  }

  // sums across the lanes that share i (x-gradient) or j (y-gradient), then one lane of each group writes
  const bool accumulate = a.accumulate != 0;
  const long long cell = cell0 + cell_local;
  const int n2p = 1 << a.lg_n2p, U = 1 << a.log2_u;
  for (int r = 0; r < r1; r++) {
    float2 v[1] = {accx[r * 64 + lane]};
    if (!DIAG) group_sum(v, n2p);
    if (valid && (DIAG || j == 0)) {
      float2 *p = a.xg.ptr + cell * a.xg.sb + (long long)r * a.xg.sm + i;
      float2 o = v[0];
      if (accumulate) o.x += p->x, o.y += p->y;
      *p = o;
    }
  }
  for (int r = 0; r < r2; r++) {
    float2 v[1] = {accy[r * 64 + lane]};
    if (!DIAG) stride_sum(v, n2p, U);
    if (valid && (DIAG || i == 0)) {
      float2 *p = a.yg.ptr + cell * a.yg.sb + (long long)r * a.yg.sm + j;
      float2 o = v[0];
      if (accumulate) o.x += p->x, o.y += p->y;
      *p = o;
    }
  }
}

// ---- host side ---------------------------------------------------------------------------------------------------

struct Tables {
  float *coef;
  int *mstart;
};
std::mutex g_mutex;
std::map<std::vector<int>, Tables> g_tables;  // (device, l1, l2, lmin, lt, present mask...) -> device tables
int g_enable = 1;

int device_tables(int l1, int l2, int lmin, int lt, const std::vector<int> &present, Tables *out) {
  int dev = 0;
  GELIB_HIP_TRY(hipGetDevice(&dev));
  std::vector<int> key = {dev, l1, l2, lmin, lt};
  key.insert(key.end(), present.begin(), present.end());
  std::lock_guard<std::mutex> lock(g_mutex);
  auto it = g_tables.find(key);
  if (it == g_tables.end()) {
    std::vector<std::vector<float>> C(kNL);
    for (int dl = 0; dl < kNL; dl++)
      if (present[dl]) {
        C[dl].resize((size_t)(2 * l1 + 1) * (2 * l2 + 1));
        cg_matrix_host(l1, l2, lmin + dl, C[dl].data());
      }
    std::vector<float> coef;
    std::vector<int> mstart;
    int step = 0;
    for (int m = -lt; m <= lt; m++) {
      mstart.push_back(step);
      const int m1lo = std::max(-l1, m - l2), m1hi = std::min(l1, m + l2);
      for (int m1 = m1lo; m1 <= m1hi; m1++, step++) {
        const int m2 = m - m1;
        for (int dl = 0; dl < kRecord; dl++) {
          float c = 0.f;
          if (dl < kNL && present[dl] && lmin + dl >= std::abs(m)) c = C[dl][(size_t)(m1 + l1) * (2 * l2 + 1) + (m2 + l2)];
          coef.push_back(c);
        }
      }
    }
    mstart.push_back(step);
    coef.insert(coef.end(), 64 * 8, 0.f);  // a wave fetches 512 floats from the first record of an m on
    Tables t{nullptr, nullptr};
    GELIB_HIP_TRY(hipMalloc((void **)&t.coef, coef.size() * sizeof(float)));
    GELIB_HIP_TRY(hipMalloc((void **)&t.mstart, mstart.size() * sizeof(int)));
    GELIB_HIP_TRY(hipMemcpy(t.coef, coef.data(), coef.size() * sizeof(float), hipMemcpyHostToDevice));
    GELIB_HIP_TRY(hipMemcpy(t.mstart, mstart.data(), mstart.size() * sizeof(int), hipMemcpyHostToDevice));
    it = g_tables.emplace(key, t).first;
  }
  *out = it->second;
  return GELIB_HIP_OK;
}

}  // namespace

int onepair_vec_bwd(const VecPlan &plan, const std::vector<const gelib_part_desc *> &g,
                    const std::vector<const gelib_part_desc *> &x, const std::vector<const gelib_part_desc *> &y,
                    const std::vector<const gelib_part_desc *> &xg, const std::vector<const gelib_part_desc *> &yg,
                    bool accumulate, hipStream_t s, int *used, bool dry_run) {
  *used = 0;
  if (!g_enable || x.size() != 1 || y.size() != 1 || xg.size() != 1 || yg.size() != 1 || plan.triples.empty())
    return GELIB_HIP_OK;
  std::vector<FastPart> fx, fy, fg, fxg, fyg;
  std::vector<std::pair<int, int>> lx, ly, lg;
  if (!lists_to_fast(x, plan.E, false, &fx, &lx) || !lists_to_fast(y, plan.E, false, &fy, &ly) ||
      !lists_to_fast(g, plan.E, false, &fg, &lg) || !lists_to_fast(xg, plan.E, true, &fxg, nullptr) ||
      !lists_to_fast(yg, plan.E, true, &fyg, nullptr))
    return GELIB_HIP_OK;
  const int l1 = lx[0].first, l2 = ly[0].first, n1 = lx[0].second, n2 = ly[0].second;
  const int lmin = std::abs(l1 - l2);
  if (2 * l1 + 1 + 2 * l2 + 1 > kMaxRows || n1 < 1 || n2 < 1) return GELIB_HIP_OK;
  int lmax = -1;
  for (auto &t : plan.triples) lmax = std::max(lmax, t.l);
  if (lmax - lmin + 1 > kNL) return GELIB_HIP_OK;
  const int lg1 = ilog2(n1), lg2 = plan.diag ? 0 : ilog2(n2);  // channel counts rounded up to powers of two
  if (lg1 + lg2 > 6) return GELIB_HIP_OK;
  OnePairArgs a;
  std::memset(&a, 0, sizeof(a));
  a.x = fx[0];
  a.y = fy[0];
  a.xg = fxg[0];
  a.yg = fyg[0];
  std::vector<int> present(kNL, 0);
  for (auto &t : plan.triples) {
    const int dl = t.l - lmin;
    a.g[dl] = fg[t.ri];
    a.offs[dl] = t.offs;
    present[dl] = 1;
  }
  const long long ncells = plan.E[0] * plan.E[1] * plan.E[2];
  const long long cpw = 64 >> (lg1 + lg2);
  for (int dl = 0; dl < kNL; dl++)  // the lane's offset inside a part must fit 32 bits
    if (present[dl] && ((cpw - 1) * a.g[dl].sb + a.g[dl].n) * 8 >= (1LL << 31)) return GELIB_HIP_OK;
  Tables t;
  const int lt = std::min(l1 + l2, lmax);
  int rc = device_tables(l1, l2, lmin, lt, present, &t);
  if (rc) return rc;
  a.coef = t.coef;
  a.mstart = t.mstart;
  a.ncells = ncells;
  a.l1 = l1;
  a.l2 = l2;
  a.lmin = lmin;
  a.lt = lt;
  a.n1 = n1;
  a.n2 = n2;
  a.log2_u = lg1 + lg2;
  a.lg_n2p = lg2;
  a.diag = plan.diag ? 1 : 0;
  a.accumulate = accumulate ? 1 : 0;
  const long long nblocks = (ncells + cpw - 1) / cpw;
  if (nblocks > 0x7fffffffLL) return GELIB_HIP_OK;
  long long lds_f2 = (2 * l1 + 1 + 2 * l2 + 1) * 64 + cpw * ((2 * l1 + 1) * n1 + (2 * l2 + 1) * n2);
  lds_f2 = (lds_f2 + 1) & ~1LL;
  a.rec_off = (int)lds_f2;
  const size_t lds = (size_t)lds_f2 * sizeof(float2) + (size_t)std::max(kStepsMax * kRecord, 64 * 8) * sizeof(float);
  if (lds > 64 * 1024) return GELIB_HIP_OK;
  if (dry_run) {  // the caller only asks whether this pair is one the kernel takes
    *used = 1;
    return GELIB_HIP_OK;
  }
  if (plan.diag) hipLaunchKernelGGL(onepair_bwd_kernel<true>, dim3((unsigned)nblocks), dim3(64), lds, s, a);
  else hipLaunchKernelGGL(onepair_bwd_kernel<false>, dim3((unsigned)nblocks), dim3(64), lds, s, a);
  GELIB_HIP_TRY(hipGetLastError());
  *used = 1;
  return GELIB_HIP_OK;
}

int onepair_set_option(const char *name, int value) {
  if (!std::strcmp(name, "onepair")) {
    g_enable = value;
    return GELIB_HIP_OK;
  }
  return GELIB_HIP_ERR_ARG;
}

}  // namespace gelib_hip
