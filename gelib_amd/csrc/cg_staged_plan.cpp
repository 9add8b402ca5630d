// Host side of the staged (any-l) kernels: eligibility, the per-signature device tables (triples + compact
// coefficient streams) and the per-call launch shape.
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <map>
#include <mutex>
#include <vector>

#include "cg_staged.h"

namespace gelib_hip {

namespace {

int g_fwd_enable = 1;
int g_bwd_enable = 1;
int g_fwd_tile = 0;           // 0 = widest tile that fits, else force 1 / 2 / 4 (still subject to divisibility)
int g_fwd_coeffs_lds = 1;     // forward coefficients staged in LDS when they fit
int g_fwd_threads = 0;        // 0 = choose from the LDS footprint
int g_bwd_stripes = 1;       // striped (register-accumulating) backward kernels: 0 never, otherwise wherever they apply
int g_bwd_atomic = 0;        // single-pass backward kernels that add partial sums into LDS with float atomics (results
                             // depend on timing in their last bits): 1 where the striped kernels do not apply, 0 never
                             // (such products then run on the shape-agnostic kernels, in a fixed order)
int g_bwd_pairs = 0;         // pair-wise single-pass backward kernel where the striped ones are not used: 1 yes, 0 no
                             // (off: measured slower than the triple-wise kernel, 6.5 vs 5.9 ms at l1 = l2 = 10)
int g_bwd_threads = 0;       // 0 = choose from the LDS footprint, else force 256 / 512 / 1024
int g_fwd_lds_target = 32 * 1024;  // LDS up to which a forward block takes more cells to fill its waves
int g_bwd_lds_target = 40 * 1024;

constexpr int kLdsLimit = 160 * 1024;

struct DevicePlan {
  std::vector<StagedTriple> triples;
  StagedTriple *d_triples = nullptr;
  float *d_bank = nullptr;
  int *d_stripes = nullptr;
  int xsize = 0, ysize = 0;
  int lmax_out = 0;
  int fwd_len = 0;           // floats of the forward coefficient stream (the first region of the bank)
  bool stripes_ok = false;   // the striped backward kernels apply
  bool stripes_skip_parts = false;  // ... but only when accumulating: some gradient part gets nothing from these triples
                                    // and would stay unwritten
  int stripe_cap = 0;        // register rows they need (16 or 32)
  std::vector<int> stripes;  // host copy of the table
  int npairs = 0;            // (x part, y part) pairs; their table follows the stripe tables
  bool pairs_ok = false;     // the pair-wise backward kernel applies
  int pair_cap = 0;          // register rows it needs (16 or 32)
  int pair_off = 0;          // ints from the start of the stripe tables to the pair table
};

std::mutex g_plan_mutex;
std::map<std::vector<int>, DevicePlan> g_plans;  // key starts with the device ordinal

// xs / ys: (l, n) of the operand parts in list order; rls: l of the product parts in list order
int get_plan(bool diag, const std::vector<VecTriple> &triples, const std::vector<std::pair<int, int>> &xs,
             const std::vector<std::pair<int, int>> &ys, const std::vector<int> &rls, const DevicePlan **out) {
  int dev = 0;
  GELIB_HIP_TRY(hipGetDevice(&dev));
  std::vector<int> key = {dev, diag ? 1 : 0, (int)xs.size(), (int)ys.size(), (int)rls.size()};
  for (auto &v : xs) key.push_back(v.first), key.push_back(v.second);
  for (auto &v : ys) key.push_back(v.first), key.push_back(v.second);
  for (int l : rls) key.push_back(l);
  for (auto &t : triples) key.push_back(t.xi), key.push_back(t.yi), key.push_back(t.ri), key.push_back(t.offs);
  std::lock_guard<std::mutex> lock(g_plan_mutex);
  auto it = g_plans.find(key);
  if (it != g_plans.end()) {
    *out = &it->second;
    return GELIB_HIP_OK;
  }
  DevicePlan plan;
  std::vector<float> bank, fwd, back0, back1, pairwise;  // the streams are laid out one after the other
  std::vector<int> xoff(xs.size()), yoff(ys.size());
  for (size_t i = 0; i < xs.size(); i++) {
    xoff[i] = plan.xsize;
    plan.xsize += (2 * xs[i].first + 1) * xs[i].second;
  }
  for (size_t i = 0; i < ys.size(); i++) {
    yoff[i] = plan.ysize;
    plan.ysize += (2 * ys[i].first + 1) * ys[i].second;
  }
  std::vector<float> full;
  for (auto &t : triples) {
    StagedTriple r;
    std::memset(&r, 0, sizeof(r));
    r.l1 = t.l1, r.l2 = t.l2, r.l = t.l;
    r.n1 = xs[t.xi].second, r.n2 = ys[t.yi].second;
    r.xi = t.xi, r.yi = t.yi, r.ri = t.ri;
    r.xoff = xoff[t.xi], r.yoff = yoff[t.yi];
    r.offs = t.offs;
    const long long U = diag ? r.n1 : (long long)r.n1 * r.n2;
    r.u = (int)U;
    {
      const int lg1 = ilog2(std::max(1, r.n1)), lg2 = ilog2(std::max(1, r.n2));
      const int lgu = diag ? lg1 : lg1 + lg2;
      r.lg_n2p = lg2;
      r.log2_u = lgu <= 20 ? lgu : -1;
    }
    const int L1 = 2 * t.l1 + 1, L2 = 2 * t.l2 + 1;
    full.assign((size_t)L1 * L2, 0.f);
    cg_matrix_host(t.l1, t.l2, t.l, full.data());
    auto C = [&](int m1, int m2) { return full[(size_t)(m1 + t.l1) * L2 + (m2 + t.l2)]; };
    r.cg_fwd = (int)fwd.size();
    for (int m = -t.l; m <= t.l; m++)
      for (int m1 = std::max(-t.l1, m - t.l2); m1 <= std::min(t.l1, m + t.l2); m1++) fwd.push_back(C(m1, m - m1));
    r.cg_back0 = (int)back0.size();
    for (int m1 = -t.l1; m1 <= t.l1; m1++)
      for (int m2 = std::max(-t.l2, -t.l - m1); m2 <= std::min(t.l2, t.l - m1); m2++) back0.push_back(C(m1, m2));
    r.cg_back1 = (int)back1.size();
    for (int m2 = -t.l2; m2 <= t.l2; m2++)
      for (int m1 = std::max(-t.l1, -t.l - m2); m1 <= std::min(t.l1, t.l - m2); m1++) back1.push_back(C(m1, m2));
    plan.lmax_out = std::max(plan.lmax_out, t.l);
    plan.triples.push_back(r);
  }
  plan.fwd_len = (int)fwd.size();
  for (auto &r : plan.triples) {
    r.cg_back0 += (int)fwd.size();
    r.cg_back1 += (int)(fwd.size() + back0.size());
  }
  // Pairs: runs of consecutive triples with the same x part and y part (their l ascending).  The pair-wise backward
  // kernel reads, for every m and every (m1, m-m1), the coefficients of all l >= |m| of the pair as one run:
  //   for m: for m1: for the pair's l >= |m| in ascending order: C_l[m1, m-m1]
  std::vector<int> pair_table;  // (first triple, count, stream offset) per pair
  {
    const int pair_base = (int)(fwd.size() + back0.size() + back1.size());
    bool ok = true;
    int rows_max = 0;
    size_t t0 = 0;
    std::vector<std::vector<float>> tabs;
    while (t0 < plan.triples.size()) {
      size_t t1 = t0 + 1;
      while (t1 < plan.triples.size() && plan.triples[t1].xi == plan.triples[t0].xi && plan.triples[t1].yi == plan.triples[t0].yi) t1++;
      const StagedTriple &f = plan.triples[t0];
      pair_table.push_back((int)t0);
      pair_table.push_back((int)(t1 - t0));
      pair_table.push_back(pair_base + (int)pairwise.size());
      rows_max = std::max({rows_max, 2 * f.l1 + 1, 2 * f.l2 + 1, (int)(t1 - t0)});
      tabs.clear();
      const int L1 = 2 * f.l1 + 1, L2 = 2 * f.l2 + 1;
      for (size_t t = t0; t < t1; t++) {
        if (t > t0 && plan.triples[t].l <= plan.triples[t - 1].l) ok = false;
        tabs.emplace_back((size_t)L1 * L2, 0.f);
        cg_matrix_host(f.l1, f.l2, plan.triples[t].l, tabs.back().data());
      }
      const int ltop = plan.triples[t1 - 1].l;
      for (int m = -ltop; m <= ltop; m++)
        for (int m1 = std::max(-f.l1, m - f.l2); m1 <= std::min(f.l1, m + f.l2); m1++)
          for (size_t t = t0; t < t1; t++)
            if (plan.triples[t].l >= std::abs(m)) pairwise.push_back(tabs[t - t0][(size_t)(m1 + f.l1) * L2 + (m - m1 + f.l2)]);
      t0 = t1;
    }
    plan.npairs = (int)pair_table.size() / 3;
    plan.pair_cap = rows_max <= 16 ? 16 : 32;
    plan.pairs_ok = ok && rows_max <= 32;
  }
  bank = fwd;
  bank.insert(bank.end(), back0.begin(), back0.end());
  bank.insert(bank.end(), back1.begin(), back1.end());
  bank.insert(bank.end(), pairwise.begin(), pairwise.end());
  bank.resize(bank.size() + 4 * kWave, 0.f);  // the kernels read the stream up to three registers of lanes ahead
  // stripes: the triples that feed one x part (resp. one y part)
  {
    const int nx = (int)xs.size(), ny = (int)ys.size(), nt = (int)plan.triples.size();
    std::vector<int> &tb = plan.stripes;
    tb.assign(3 * (nx + ny) + 2 * nt, 0);
    bool ok = true;
    int lown = 0;
    for (int role = 0; role < 2; role++) {
      const int np = role == 0 ? nx : ny;
      int *table = tb.data() + (role == 0 ? 0 : 3 * nx);
      int *order = tb.data() + 3 * (nx + ny) + (role == 0 ? 0 : nt);
      int filled = 0;
      for (int k = 0; k < np; k++) {
        const int n_own = role == 0 ? xs[k].second : ys[k].second;
        lown = std::max(lown, role == 0 ? xs[k].first : ys[k].first);
        table[3 * k] = filled;
        int n_other = -1;
        for (int t = 0; t < nt; t++) {
          const StagedTriple &r = plan.triples[t];
          if ((role == 0 ? r.xi : r.yi) != k) continue;
          order[filled++] = t;
          const int no = role == 0 ? r.n2 : r.n1;
          if (n_other >= 0 && no != n_other) ok = false;  // a lane's (i, j) would change inside the stripe
          n_other = no;
        }
        table[3 * k + 1] = filled - table[3 * k];
        // a part that no triple feeds has a zero gradient; a stripe without units leaves it as it is, which is right
        // when the call accumulates (the second half of a product split between two kernel families) and wrong when it
        // overwrites
        if (table[3 * k + 1] == 0) plan.stripes_skip_parts = true;
        // lane slots: channel counts rounded up to powers of two
        const int lgu = diag ? ilog2(std::max(1, n_own)) : ilog2(std::max(1, n_own)) + ilog2(std::max(1, n_other));
        if (lgu > 20) ok = false;
        table[3 * k + 2] = ok ? lgu : 0;
      }
    }
    if (!diag)
      for (auto &v : ys)
        if (v.second > kWave) ok = false;
    if (2 * lown + 1 > 32) ok = false;
    plan.stripes_ok = ok;
    plan.stripe_cap = 2 * lown + 1 <= 16 ? 16 : 32;
    plan.pair_off = (int)tb.size();
    tb.insert(tb.end(), pair_table.begin(), pair_table.end());
  }
  const size_t tri_bytes = plan.triples.size() * sizeof(StagedTriple);
  const size_t bank_bytes = bank.size() * sizeof(float);
  const size_t stripe_bytes = plan.stripes.size() * sizeof(int);
  char *d = nullptr;
  GELIB_HIP_TRY(hipMalloc((void **)&d, tri_bytes + bank_bytes + stripe_bytes));
  hipError_t e = hipMemcpy(d, plan.triples.data(), tri_bytes, hipMemcpyHostToDevice);
  if (e == hipSuccess) e = hipMemcpy(d + tri_bytes, bank.data(), bank_bytes, hipMemcpyHostToDevice);
  if (e == hipSuccess) e = hipMemcpy(d + tri_bytes + bank_bytes, plan.stripes.data(), stripe_bytes, hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    (void)hipFree(d);
    return record_hip_error(e, "hipMemcpy(staged plan)");
  }
  plan.d_triples = (StagedTriple *)d;
  plan.d_bank = (float *)(d + tri_bytes);
  plan.d_stripes = (int *)(d + tri_bytes + bank_bytes);
  auto ins = g_plans.emplace(key, std::move(plan));
  *out = &ins.first->second;
  return GELIB_HIP_OK;
}

struct FastLists {
  std::vector<FastPart> x, y, r, xg, yg;
};

long long units_per_block(const DevicePlan &plan, long long cpb) {
  long long units = 0;
  for (auto &t : plan.triples) units += (cpb * t.u + kWave - 1) / kWave;
  return units;
}

void fill_args(StagedArgs &a, const DevicePlan &plan, const FastLists &f, const std::vector<std::pair<int, int>> &xs,
               const std::vector<std::pair<int, int>> &ys, long long ncells, int offs_add, bool accumulate) {
  std::memset(&a, 0, sizeof(a));
  for (size_t i = 0; i < f.x.size(); i++) a.x[i] = f.x[i];
  for (size_t i = 0; i < f.y.size(); i++) a.y[i] = f.y[i];
  for (size_t i = 0; i < f.r.size(); i++) a.r[i] = f.r[i];
  for (size_t i = 0; i < f.xg.size(); i++) a.xg[i] = f.xg[i];
  for (size_t i = 0; i < f.yg.size(); i++) a.yg[i] = f.yg[i];
  a.triples = plan.d_triples;
  a.bank = plan.d_bank;
  a.stripes = plan.d_stripes;
  a.pairs = plan.d_stripes + plan.pair_off;
  a.npairs = plan.npairs;
  a.ncells = ncells;
  a.ntriples = (int)plan.triples.size();
  a.nx = (int)xs.size();
  a.ny = (int)ys.size();
  a.offs_add = offs_add;
  a.accumulate = accumulate ? 1 : 0;
  a.xsize = plan.xsize;
  a.ysize = plan.ysize;
  for (size_t i = 0; i < xs.size(); i++) a.xrows[i] = 2 * xs[i].first + 1;
  for (size_t i = 0; i < ys.size(); i++) a.yrows[i] = 2 * ys[i].first + 1;
}

bool sizes_ok(const std::vector<std::pair<int, int>> &xs, const std::vector<std::pair<int, int>> &ys,
              const std::vector<int> &rls) {
  if (xs.size() > (size_t)kStagedMaxParts || ys.size() > (size_t)kStagedMaxParts || rls.size() > (size_t)kStagedMaxOutParts) return false;
  long long xsize = 0, ysize = 0;
  for (auto &v : xs) xsize += (2LL * v.first + 1) * v.second;
  for (auto &v : ys) ysize += (2LL * v.first + 1) * v.second;
  return 8 * (xsize + ysize) <= kLdsLimit;
}

int run_fwd(bool diag, const std::vector<VecTriple> &triples, const std::vector<std::pair<int, int>> &xs,
            const std::vector<std::pair<int, int>> &ys, const std::vector<int> &rls, const FastLists &f,
            long long ncells, int offs_add, bool accumulate, hipStream_t s, int *used) {
  *used = 0;
  if (!sizes_ok(xs, ys, rls)) return GELIB_HIP_OK;
  for (auto &t : triples) {
    const long long U = diag ? xs[t.xi].second : (long long)xs[t.xi].second * ys[t.yi].second;
    if (U > (1 << 24)) return GELIB_HIP_OK;
  }
  const DevicePlan *plan = nullptr;
  int rc = get_plan(diag, triples, xs, ys, rls, &plan);
  if (rc) return rc;
  const long long cell_bytes = 8LL * (plan->xsize + plan->ysize);
  // The forward coefficient stream goes into LDS next to the operands when it fits: read from memory it would
  // share the wave's memory counter with the output stores and every refill would wait for them.
  const long long coeff_bytes = (g_fwd_coeffs_lds && 4LL * plan->fwd_len <= 64 * 1024 && cell_bytes + 4LL * plan->fwd_len <= kLdsLimit)
                                    ? 4LL * ((plan->fwd_len + 3) / 4 * 4) : 0;
  // Channels per lane: the widest tile that divides every channel count and offset and keeps the 16-byte
  // accesses aligned, provided enough cells fit in LDS to fill a wave with tile slots.
  auto tile_ok = [&](int tile) {
    if (tile == 1) return true;
    if (offs_add % tile || plan->xsize % tile || plan->ysize % tile) return false;  // images stay 16-byte aligned
    for (auto &t : plan->triples) {
      if ((diag ? t.n1 : t.n2) % tile || t.offs % tile) return false;
      if (diag && (t.xoff % tile || t.yoff % tile)) return false;
      if (t.yoff % tile) return false;
    }
    for (auto &r : f.r)
      if (((uintptr_t)r.ptr % (8 * tile)) || r.sb % tile || r.sm % tile) return false;
    return true;
  };
  int tile = 4, threads = 256;
  long long cpb = 1;
  if (g_fwd_tile == 1 || g_fwd_tile == 2 || g_fwd_tile == 4) tile = g_fwd_tile;
  for (;; tile >>= 1) {
    if (!tile_ok(tile)) continue;
    long long slots_min = 1 << 30;
    for (auto &t : plan->triples) slots_min = std::min<long long>(slots_min, t.u / tile);
    auto units = [&](long long c) {
      long long n = 0;
      for (auto &t : plan->triples) n += (c * (t.u / tile) + kWave - 1) / kWave;
      return n;
    };
    cpb = 1;
    // first fill the lanes of a run, then give the block's waves enough runs
    while (cpb * 2 <= ncells && cpb * slots_min < kWave && cell_bytes * cpb * 2 + coeff_bytes <= 140 * 1024) cpb *= 2;
    while (cpb * 2 <= ncells && cell_bytes * cpb * 2 + coeff_bytes <= g_fwd_lds_target && units(cpb) < 16) cpb *= 2;
    if (tile > 1 && cpb * slots_min < kWave && cpb < ncells) continue;  // lanes would idle: try a narrower tile
    // as many waves per CU as the LDS footprint leaves room for, without more waves than runs
    const long long blocks_per_cu = std::max<long long>(1, kLdsLimit / std::max<long long>(1, cell_bytes * cpb + coeff_bytes));
    long long waves = std::max<long long>(4, std::min<long long>(16, 32 / blocks_per_cu));
    while (waves > 4 && units(cpb) < 2 * waves) waves >>= 1;
    threads = (int)waves * kWave;
    break;
  }
  if (g_fwd_threads >= 64 && g_fwd_threads <= 1024 && g_fwd_threads % 64 == 0) threads = g_fwd_threads;
  StagedArgs a;
  fill_args(a, *plan, f, xs, ys, ncells, offs_add, accumulate);
  a.cpb = (int)cpb;
  a.lds_coeffs = coeff_bytes ? plan->fwd_len : 0;
  const long long nblocks = (ncells + cpb - 1) / cpb;
  if (nblocks > 0x7fffffffLL) return GELIB_HIP_ERR_ARG;
  rc = launch_staged_fwd(a, diag, tile, threads, (int)nblocks, (size_t)(cell_bytes * cpb + coeff_bytes), s);
  if (rc) return rc;
  *used = 1;
  return GELIB_HIP_OK;
}

int run_bwd(bool diag, const std::vector<VecTriple> &triples, const std::vector<std::pair<int, int>> &xs,
            const std::vector<std::pair<int, int>> &ys, const std::vector<int> &rls, const FastLists &f,
            long long ncells, int offs_add, bool accumulate, bool want_x, bool want_y, hipStream_t s, int *used) {
  *used = 0;
  if (!sizes_ok(xs, ys, rls)) return GELIB_HIP_OK;
  // lane slots are the channel counts rounded up to powers of two; the second operand's must fit one wave
  for (auto &t : triples) {
    const int n1 = xs[t.xi].second, n2 = ys[t.yi].second;
    if (n1 < 1 || n2 < 1) return GELIB_HIP_OK;
    if (!diag && n2 > kWave) return GELIB_HIP_OK;
    if ((diag ? ilog2(n1) : ilog2(n1) + ilog2(n2)) > 20) return GELIB_HIP_OK;
  }
  const DevicePlan *plan = nullptr;
  int rc = get_plan(diag, triples, xs, ys, rls, &plan);
  if (rc) return rc;
  // The striped kernels sum in a fixed order and win where rows are short; with 32 register rows for g and 32 for the
  // sums (own l above 7) they run at low occupancy, still 2.7 times faster than the atomic single-pass form on vectors
  // of several parts around l = 10 (6.7 against 18.4 ms; the per-pair route of the dispatcher takes those first).
  const bool stripes_wanted = g_bwd_stripes != 0;
  if (stripes_wanted && plan->stripes_ok && (accumulate || !plan->stripes_skip_parts) &&
      8LL * std::max(plan->xsize, plan->ysize) + 64 <= kLdsLimit) {
    // one launch per wanted gradient; LDS holds the other operand only
    StagedArgs a;
    fill_args(a, *plan, f, xs, ys, ncells, offs_add, accumulate);
    for (int role = 0; role < 2; role++) {
      if (role == 0 ? !want_x : !want_y) continue;
      const long long cell_bytes = 8LL * (role == 0 ? plan->ysize : plan->xsize);
      const int np = role == 0 ? (int)xs.size() : (int)ys.size();
      const int *table = plan->stripes.data() + (role == 0 ? 0 : 3 * (int)xs.size());
      auto units = [&](long long cpb) {
        long long n = 0;
        for (int k = 0; k < np; k++) {
          const int lg = table[3 * k + 2];
          n += lg >= 6 ? cpb : (((cpb << lg) + kWave - 1) >> 6);
        }
        return n;
      };
      long long cpb = 1;
      while (cpb * 2 <= ncells && cell_bytes * cpb * 2 <= g_bwd_lds_target && units(cpb) < 16) cpb *= 2;
      a.cpb = (int)cpb;
      const long long nblocks = (ncells + cpb - 1) / cpb;
      if (nblocks > 0x7fffffffLL) return GELIB_HIP_ERR_ARG;
      rc = launch_staged_stripe(a, diag, role, plan->stripe_cap, (int)nblocks, (size_t)(cell_bytes * cpb), s);
      if (rc) return rc;
    }
    *used = 1;
    return GELIB_HIP_OK;
  }
  if (!g_bwd_atomic) return GELIB_HIP_OK;  // what is left adds with float atomics: only on request
  const long long cell_bytes = 16LL * (plan->xsize + plan->ysize);  // operands + gradient images
  if (cell_bytes > kLdsLimit) return GELIB_HIP_OK;
  // n2 <= 64 and power-of-two channel counts hold here; the pair-wise kernel also needs uniform slots per pair,
  // which one pair always has
  if (g_bwd_pairs && plan->pairs_ok) {
    auto units = [&](long long c) {
      long long n = 0;
      for (int k = 0; k < plan->npairs; k++)
        n += ((c << plan->triples[plan->stripes[plan->pair_off + 3 * k]].log2_u) + kWave - 1) / kWave;
      return n;
    };
    long long cpb = 1;
    while (cpb * 2 <= ncells && cell_bytes * cpb * 2 <= g_bwd_lds_target && units(cpb) < 8) cpb *= 2;
    StagedArgs a;
    fill_args(a, *plan, f, xs, ys, ncells, offs_add, accumulate);
    a.cpb = (int)cpb;
    const long long nblocks = (ncells + cpb - 1) / cpb;
    if (nblocks > 0x7fffffffLL) return GELIB_HIP_ERR_ARG;
    rc = launch_staged_pair_bwd(a, diag, want_x, want_y, plan->pair_cap, (int)nblocks, (size_t)(cell_bytes * cpb), s);
    if (rc) return rc;
    *used = 1;
    return GELIB_HIP_OK;
  }
  long long cpb = 1;
  while (cpb * 2 <= ncells && cell_bytes * cpb * 2 <= g_bwd_lds_target && units_per_block(*plan, cpb) < 16) cpb *= 2;
  const long long lds = cell_bytes * cpb;
  const int rows = 2 * plan->lmax_out + 1;
  const int cap = rows <= 16 ? 16 : 32;
  const int max_threads = cap == 16 ? 1024 : 512;
  int threads = 256;
  const long long units = units_per_block(*plan, cpb);
  if (lds > 52 * 1024 && units >= 16) threads = 512;       // at most two blocks fit a CU: make them wider
  if (lds > 80 * 1024 && units >= 32) threads = 1024;      // one block per CU
  if (g_bwd_threads == 256 || g_bwd_threads == 512 || g_bwd_threads == 1024) threads = g_bwd_threads;
  threads = std::min(threads, max_threads);
  StagedArgs a;
  fill_args(a, *plan, f, xs, ys, ncells, offs_add, accumulate);
  a.cpb = (int)cpb;
  const long long nblocks = (ncells + cpb - 1) / cpb;
  if (nblocks > 0x7fffffffLL) return GELIB_HIP_ERR_ARG;
  rc = launch_staged_bwd(a, diag, want_x, want_y, cap, threads, (int)nblocks, (size_t)lds, s);
  if (rc) return rc;
  *used = 1;
  return GELIB_HIP_OK;
}

}  // namespace

int staged_part(int kind, const PartOp &op, bool accumulate, hipStream_t s, int *used) {
  *used = 0;
  if (kind == 0 && !g_fwd_enable) return GELIB_HIP_OK;
  if (kind != 0 && !g_bwd_enable) return GELIB_HIP_OK;
  FastLists f;
  f.x.resize(1);
  f.y.resize(1);
  f.r.resize(1);
  if (!to_fast(op.r, op.E, op.Dr, op.offs + op.nout, kind == 0, &f.r[0])) return GELIB_HIP_OK;
  if (!to_fast(op.x, op.E, op.Dx, op.n1, kind == 1, &f.x[0])) return GELIB_HIP_OK;
  if (!to_fast(op.y, op.E, op.Dy, op.n2, kind == 2, &f.y[0])) return GELIB_HIP_OK;
  const long long ncells = op.E[0] * op.E[1] * op.E[2];
  std::vector<VecTriple> triples = {{0, 0, 0, op.l1, op.l2, op.l, 0, op.nout}};
  std::vector<std::pair<int, int>> xs = {{op.l1, op.n1}}, ys = {{op.l2, op.n2}};
  std::vector<int> rls = {op.l};
  if (kind == 0) return run_fwd(op.diag, triples, xs, ys, rls, f, ncells, op.offs, accumulate, s, used);
  if (kind == 1) f.xg = f.x;  // destination
  if (kind == 2) f.yg = f.y;
  return run_bwd(op.diag, triples, xs, ys, rls, f, ncells, op.offs, accumulate, kind == 1, kind == 2, s, used);
}

int staged_vec_fwd(const VecPlan &plan, const std::vector<const gelib_part_desc *> &r,
                   const std::vector<const gelib_part_desc *> &x, const std::vector<const gelib_part_desc *> &y,
                   bool accumulate, hipStream_t s, int *used) {
  *used = 0;
  if (!g_fwd_enable) return GELIB_HIP_OK;
  FastLists f;
  std::vector<std::pair<int, int>> xs, ys, rs;
  if (!lists_to_fast(x, plan.E, false, &f.x, &xs) || !lists_to_fast(y, plan.E, false, &f.y, &ys) ||
      !lists_to_fast(r, plan.E, true, &f.r, &rs))
    return GELIB_HIP_OK;
  std::vector<int> rls;
  for (auto &v : rs) rls.push_back(v.first);
  const long long ncells = plan.E[0] * plan.E[1] * plan.E[2];
  return run_fwd(plan.diag, plan.triples, xs, ys, rls, f, ncells, 0, accumulate, s, used);
}

int staged_vec_bwd(const VecPlan &plan, const std::vector<const gelib_part_desc *> &g,
                   const std::vector<const gelib_part_desc *> &x, const std::vector<const gelib_part_desc *> &y,
                   const std::vector<const gelib_part_desc *> &xg, const std::vector<const gelib_part_desc *> &yg,
                   bool accumulate, hipStream_t s, int *used) {
  *used = 0;
  if (!g_bwd_enable) return GELIB_HIP_OK;
  FastLists f;
  std::vector<std::pair<int, int>> xs, ys, rs;
  if (!lists_to_fast(x, plan.E, false, &f.x, &xs) || !lists_to_fast(y, plan.E, false, &f.y, &ys) ||
      !lists_to_fast(g, plan.E, false, &f.r, &rs))
    return GELIB_HIP_OK;
  if (!xg.empty() && !lists_to_fast(xg, plan.E, true, &f.xg, nullptr)) return GELIB_HIP_OK;
  if (!yg.empty() && !lists_to_fast(yg, plan.E, true, &f.yg, nullptr)) return GELIB_HIP_OK;
  std::vector<int> rls;
  for (auto &v : rs) rls.push_back(v.first);
  const long long ncells = plan.E[0] * plan.E[1] * plan.E[2];
  return run_bwd(plan.diag, plan.triples, xs, ys, rls, f, ncells, 0, accumulate, !xg.empty(), !yg.empty(), s, used);
}

int staged_set_option(const char *name, int value) {
  if (!std::strcmp(name, "staged_fwd")) {
    g_fwd_enable = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "staged_bwd")) {
    g_bwd_enable = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "staged_fwd_tile")) {
    g_fwd_tile = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "staged_fwd_coeffs_lds")) {
    g_fwd_coeffs_lds = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "staged_fwd_threads")) {
    g_fwd_threads = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "staged_bwd_stripes")) {
    g_bwd_stripes = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "staged_bwd_atomic")) {
    g_bwd_atomic = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "staged_bwd_pairs")) {
    g_bwd_pairs = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "staged_bwd_threads")) {
    if (value != 0 && value != 256 && value != 512 && value != 1024) return GELIB_HIP_ERR_ARG;
    g_bwd_threads = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "staged_fwd_lds_target")) {
    if (value < 1024 || value > kLdsLimit) return GELIB_HIP_ERR_ARG;
    g_fwd_lds_target = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "staged_bwd_lds_target")) {
    if (value < 1024 || value > kLdsLimit) return GELIB_HIP_ERR_ARG;
    g_bwd_lds_target = value;
    return GELIB_HIP_OK;
  }
  return GELIB_HIP_ERR_ARG;
}

}  // namespace gelib_hip
