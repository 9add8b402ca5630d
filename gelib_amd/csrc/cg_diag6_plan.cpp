// Host side of the lane-per-channel Diag kernels: which products they take, the coefficient table with its fixed
// layout, the per-type offset table (both cached on the device), and the argument block.
#include <algorithm>
#include <cstring>
#include <map>
#include <mutex>
#include <vector>

#include "cg_diag6.h"

namespace gelib_hip {

namespace {

// ---- host side ---------------------------------------------------------------------------------------------------

std::mutex g_mutex;
std::map<int, float *> g_banks;                     // device -> coefficient table
std::map<std::pair<int, std::vector<int>>, int *> g_offs;  // (device, offsets) -> device copy
int g_enable = 1;
int g_l8_enable = 1;    // the kernels for products up to l = 8 of operands up to l = 4: 1 forward, 2 backward too
int g_sets_enable = 1;  // backward: the kernel with the waves' sets of l2 fixed at compile time, where it applies
int g_small_enable = 1;  // operands up to l = 2, and backward up to l = 4: the kernels that give a wave, not a block, a cell and
                         // channel group
int g_hi_enable = 1;    // the kernels for the part l = 7..12 of a product by itself
int g_one_channel = 1;  // CGproduct with a one-channel operand runs here as the Diag product with the channel repeated

int device_bank(const float **out) {
  int dev = 0;
  GELIB_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_mutex);
  auto it = g_banks.find(dev);
  if (it == g_banks.end()) {
    std::vector<float> h((size_t)kBankFloats + kZeroFloats, 0.f);
    for (int a = 0; a <= kL6; a++)
      for (int b = 0; b <= kL6; b++)
        for (int c = iabs(a - b); c <= a + b; c++) cg_matrix_host(a, b, c, h.data() + table_off(a, b, c));
    float *d = nullptr;
    GELIB_HIP_TRY(hipMalloc((void **)&d, h.size() * sizeof(float)));
    GELIB_HIP_TRY(hipMemcpy(d, h.data(), h.size() * sizeof(float), hipMemcpyHostToDevice));
    it = g_banks.emplace(dev, d).first;
  }
  *out = it->second;
  return GELIB_HIP_OK;
}

int device_offs(const std::vector<int> &h, const int **out) {
  int dev = 0;
  GELIB_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_mutex);
  auto key = std::make_pair(dev, h);
  auto it = g_offs.find(key);
  if (it == g_offs.end()) {
    int *d = nullptr;
    GELIB_HIP_TRY(hipMalloc((void **)&d, h.size() * sizeof(int)));
    GELIB_HIP_TRY(hipMemcpy(d, h.data(), h.size() * sizeof(int), hipMemcpyHostToDevice));
    it = g_offs.emplace(key, d).first;
  }
  *out = it->second;
  return GELIB_HIP_OK;
}

// Fills the argument block; *ok = false when the product is not one this family takes.
int make_args(const VecPlan &plan, const std::vector<const gelib_part_desc *> &r,
              const std::vector<const gelib_part_desc *> &x, const std::vector<const gelib_part_desc *> &y,
              const std::vector<const gelib_part_desc *> *xg, const std::vector<const gelib_part_desc *> *yg,
              bool r_is_dest, Diag6Args *a, int *lcap, bool *ok, int *llo = nullptr) {
  *ok = false;
  if (!g_enable) return GELIB_HIP_OK;
  std::vector<FastPart> fx, fy, fr, fxg, fyg;
  std::vector<std::pair<int, int>> lx, ly, lr;
  if (!lists_to_fast(x, plan.E, false, &fx, &lx) || !lists_to_fast(y, plan.E, false, &fy, &ly) ||
      !lists_to_fast(r, plan.E, r_is_dest, &fr, &lr))
    return GELIB_HIP_OK;
  if (xg && !lists_to_fast(*xg, plan.E, true, &fxg, nullptr)) return GELIB_HIP_OK;
  if (yg && !lists_to_fast(*yg, plan.E, true, &fyg, nullptr)) return GELIB_HIP_OK;
  // A CGproduct in which every part of one operand has ONE channel is the Diag product with that channel repeated:
  // block channel i * 1 + 0 (resp. 0 * n + j) is the wide operand's own channel, and the blocks follow each other n
  // apart either way (core/Gvec.hpp:311-321 against :358-367).  Lanes then all read the one channel, and its gradient
  // is a sum over the lanes of a cell (one block per cell: up to 64 channels).
  bool xbc = false, ybc = false;
  if (!plan.diag) {
    if (!g_one_channel) return GELIB_HIP_OK;
    auto all_one = [](const std::vector<std::pair<int, int>> &v) {
      for (auto &p : v)
        if (p.second != 1) return false;
      return true;
    };
    ybc = all_one(ly);
    xbc = all_one(lx);
    if (xbc && ybc && !xg && !yg) {
      // one channel on both sides, forward: block channel 0 * 1 + 0 -- the Diag product of one channel, a cell per lane
      // (the gradients of such a product stay with the unrolled kernels, which are faster there)
      xbc = ybc = false;
    } else if (xbc == ybc) {
      return GELIB_HIP_OK;   // otherwise exactly one narrow side
    }
  }
  const int n = (xbc ? ly : lx)[0].second;
  if (n < 1 || n > kMaxChannels) return GELIB_HIP_OK;
  if ((xbc && xg && n > 64) || (ybc && yg && n > 64)) return GELIB_HIP_OK;
  for (auto &p : lx)
    if (p.first > kL6 || p.second != (xbc ? 1 : n)) return GELIB_HIP_OK;
  for (auto &p : ly)
    if (p.first > kL6 || p.second != (ybc ? 1 : n)) return GELIB_HIP_OK;
  for (auto &p : lr)
    if (p.first > 2 * kL6) return GELIB_HIP_OK;
  std::memset(a, 0, sizeof(*a));
  for (size_t i = 0; i < fx.size(); i++) a->x[lx[i].first] = fx[i];
  for (size_t i = 0; i < fy.size(); i++) a->y[ly[i].first] = fy[i];
  for (size_t i = 0; i < fr.size(); i++) a->r[lr[i].first] = fr[i];
  for (size_t i = 0; i < fxg.size(); i++) a->xg[lx[i].first] = fxg[i];
  for (size_t i = 0; i < fyg.size(); i++) a->yg[ly[i].first] = fyg[i];
  {
    // Deal the parts of y to the four waves of a backward block, heaviest first, each to the wave with the least work so
    // far, so that the waves finish every l1 at about the same time.  Work of a pair: two multiply-adds per term of each
    // of its triples (the contraction over l) and eight per (m1, m2).
    long long cost[kNP] = {0, 0, 0, 0, 0, 0, 0};
    bool pair_seen[kNP][kNP] = {};
    for (auto &t : plan.triples) {
      long long terms = 0;
      for (int m = -t.l; m <= t.l; m++) terms += std::min(t.l1, m + t.l2) - std::max(-t.l1, m - t.l2) + 1;
      cost[t.l2] += 2 * terms;
      if (!pair_seen[t.l1][t.l2]) {
        pair_seen[t.l1][t.l2] = true;
        cost[t.l2] += 8LL * (2 * t.l1 + 1) * (2 * t.l2 + 1);
      }
    }
    long long load[4] = {0, 0, 0, 0};
    bool dealt[kNP] = {};
    for (int n = 0; n < kNP; n++) {
      int best = -1;
      for (int l2 = 0; l2 < kNP; l2++)
        if (!dealt[l2] && (best < 0 || cost[l2] > cost[best])) best = l2;
      dealt[best] = true;
      int w = 0;
      for (int k = 1; k < 4; k++)
        if (load[k] < load[w]) w = k;
      a->owner[best] = w;
      load[w] += cost[best];
    }
  }
  std::vector<int> offs((size_t)kNP * kNP * kNR, -1);
  *lcap = 0;
  int lowest = 1 << 30;
  for (auto &t : plan.triples) {
    offs[((size_t)t.l1 * kNP + t.l2) * kNR + t.l] = t.offs;
    *lcap = std::max(*lcap, t.l);
    lowest = std::min(lowest, t.l);
  }
  if (llo) *llo = lowest;
  int rc = device_offs(offs, &a->offs);
  if (rc) return rc;
  if ((rc = device_bank(&a->bank))) return rc;
  const long long ncells = plan.E[0] * plan.E[1] * plan.E[2];
  a->ncells = ncells;
  a->n = n;
  a->xbc = xbc ? 1 : 0;
  a->ybc = ybc ? 1 : 0;
  int lg = 0;
  while ((1 << lg) < n && lg < 6) lg++;
  a->lg_npad = lg;
  if (lg < 6) {
    // several cells per wave: the lane's offset from the wave's first cell must fit 32 bits in every part
    const long long cpw = 64 >> lg;
    auto fits = [&](const std::vector<FastPart> &v) {
      for (auto &p : v)
        if (p.sb < 0 || ((cpw - 1) * p.sb + n) * 8 >= (1LL << 31)) return false;
      return true;
    };
    if (!fits(fx) || !fits(fy) || !fits(fr) || !fits(fxg) || !fits(fyg)) return GELIB_HIP_OK;
    a->groups = 1;
    a->nwaves = (ncells + cpw - 1) / cpw;
  } else {
    a->groups = (n + 63) / 64;
    a->nwaves = ncells * a->groups;
  }
  if (a->nwaves > 0x7fffffffLL) return GELIB_HIP_OK;
  *ok = true;
  return GELIB_HIP_OK;
}

}  // namespace

int cg_table_bank(const float **out) { return device_bank(out); }

namespace {
// no operand part (and no gradient of one) above l = lmax
bool operands_up_to(const Diag6Args &a, int lmax) {
  for (int l = lmax + 1; l < kNP; l++)
    if (a.x[l].ptr || a.y[l].ptr || a.xg[l].ptr || a.yg[l].ptr) return false;
  return true;
}
}  // namespace

int diag6_vec_fwd(const VecPlan &plan, const std::vector<const gelib_part_desc *> &r,
                  const std::vector<const gelib_part_desc *> &x, const std::vector<const gelib_part_desc *> &y,
                  bool accumulate, hipStream_t s, int *used) {
  *used = 0;
  Diag6Args a;
  int lcap = 0, llo = 0;
  bool ok = false;
  int rc = make_args(plan, r, x, y, nullptr, nullptr, true, &a, &lcap, &ok, &llo);
  if (rc || !ok) return rc;
  // kernels are built for products capped at l = 6, for products up to l = 8 of operands up to l = 4, and for the part
  // l = 7..12 of a product by itself
  const bool hi = llo > kL6 && g_hi_enable;
  const bool l8 = lcap > kL6 && !hi;
  if (l8 && !(lcap <= 8 && operands_up_to(a, 4) && g_l8_enable)) return GELIB_HIP_OK;
  a.accumulate = accumulate ? 1 : 0;
  if (g_small_enable && lcap <= 4 && operands_up_to(a, 2)) rc = launch_diag6_small_fwd(a, s);
  else if (hi) rc = a.lg_npad < 6 ? launch_diag6_fwd_hi_packed(a, s) : launch_diag6_fwd_hi(a, s);
  else if (l8) rc = a.lg_npad < 6 ? launch_diag6_fwd_l8_packed(a, s) : launch_diag6_fwd_l8(a, s);
  else rc = a.lg_npad < 6 ? launch_diag6_fwd_l6_packed(a, s) : launch_diag6_fwd_l6(a, s);
  if (rc) return rc;
  *used = 1;
  return GELIB_HIP_OK;
}

int diag6_vec_bwd(const VecPlan &plan, const std::vector<const gelib_part_desc *> &g,
                  const std::vector<const gelib_part_desc *> &x, const std::vector<const gelib_part_desc *> &y,
                  const std::vector<const gelib_part_desc *> &xg, const std::vector<const gelib_part_desc *> &yg,
                  bool accumulate, hipStream_t s, int *used) {
  *used = 0;
  if (xg.empty() && yg.empty()) return GELIB_HIP_OK;
  Diag6Args a;
  int lcap = 0, llo = 0;
  bool ok = false;
  int rc = make_args(plan, g, x, y, xg.empty() ? nullptr : &xg, yg.empty() ? nullptr : &yg, false, &a, &lcap, &ok, &llo);
  if (rc || !ok) return rc;
  // (backward, the one-launch kernel for products up to l = 8 is used on request only, diag6_l8 = 2: the wave that owns
  // y[4] then has the terms of l = 5..8 on top of the largest share, and L=4, 64 channels, 131072 cells takes 16.4 ms
  // against 14.4 ms for the split at l = 6)
  const bool hi = llo > kL6 && g_hi_enable;
  const bool l8 = lcap > kL6 && !hi;
  if (l8 && !(lcap <= 8 && operands_up_to(a, 4) && g_l8_enable >= 2)) return GELIB_HIP_OK;
  a.accumulate = accumulate ? 1 : 0;
  a.want_x = xg.empty() ? 0 : 1;
  a.want_y = yg.empty() ? 0 : 1;
  bool all_y = true;
  for (int l = 0; l < kNP; l++) all_y = all_y && a.y[l].ptr != nullptr;
  if (g_small_enable && lcap <= 4 && operands_up_to(a, 2)) rc = launch_diag6_small_bwd(a, s);
  else if (g_small_enable && hi && lcap <= 8 && operands_up_to(a, 4)) rc = launch_diag6_small4_hi_bwd(a, s);
  else if (g_small_enable && lcap <= 6 && operands_up_to(a, 4)) rc = launch_diag6_small4_bwd(a, s);
  else if (hi) rc = a.lg_npad < 6 ? launch_diag6_bwd_hi_packed(a, s) : launch_diag6_bwd_hi(a, s);
  else if (l8) rc = a.lg_npad < 6 ? launch_diag6_bwd_l8_packed(a, s) : launch_diag6_bwd_l8(a, s);
  else if (a.lg_npad < 6) rc = launch_diag6_bwd_l6_packed(a, s);
  else if (all_y && g_sets_enable) rc = launch_diag6_bwd_l6_sets(a, s);
  else rc = launch_diag6_bwd_l6(a, s);
  if (rc) return rc;
  *used = 1;
  return GELIB_HIP_OK;
}

// One triple (the part-level entry points).  kind 0: r += x * y; 1: the x-shaped tensor is the gradient wanted, r is the
// incoming gradient and the x operand does not exist; 2: likewise for y.  The missing operand is stood in for by the
// gradient's own descriptor: it only marks the part as present, the kernel never reads an operand whose gradient is
// not wanted.
int diag6_part(int kind, const long long E[3], const gelib_part_desc *r, const gelib_part_desc *x,
               const gelib_part_desc *y, int l1, int l2, int l, int offs, bool accumulate, hipStream_t s, int *used) {
  *used = 0;
  VecPlan plan;
  plan.diag = true;
  for (int k = 0; k < 3; k++) plan.E[k] = E[k];
  VecTriple t;
  t.xi = t.yi = t.ri = 0;
  t.l1 = l1;
  t.l2 = l2;
  t.l = l;
  t.offs = offs;
  t.nout = (int)x->dims[4];
  plan.triples.push_back(t);
  const std::vector<const gelib_part_desc *> R = {r}, X = {x}, Y = {y}, none;
  if (kind == 0) return diag6_vec_fwd(plan, R, X, Y, accumulate, s, used);
  return diag6_vec_bwd(plan, R, X, Y, kind == 1 ? X : none, kind == 2 ? Y : none, accumulate, s, used);
}

int diag6_set_option(const char *name, int value) {
  if (!std::strcmp(name, "diag6")) {
    g_enable = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "diag6_small")) {
    g_small_enable = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "diag6_hi")) {
    g_hi_enable = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "diag6_l8")) {
    g_l8_enable = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "diag6_one_channel")) {
    g_one_channel = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "diag6_sets")) {
    g_sets_enable = value;
    return GELIB_HIP_OK;
  }
  return GELIB_HIP_ERR_ARG;
}

}  // namespace gelib_hip
