// Host side of the unrolled small-l kernels: eligibility, collapsing (batch, grid0, grid1) into one cell index,
// the per-signature device tables (pairs + coefficient bank) and the per-call block schedule.
#include <algorithm>
#include <cstring>
#include <map>
#include <mutex>
#include <vector>

#include "cg_unrolled_dev.h"

namespace gelib_hip {

namespace {

int g_fwd_block_bytes = 0;           // product bytes one forward block aims to write (0 = by the largest l of the product)
int g_fwd_lds_bytes = 16 * 1024;     // LDS one forward block may use for its staged operands
int g_fwd_cell_tile = -1;            // cells per tile of the forward launch (0 = all cells in one tile, -1 = by channels)
int g_fwd_narrow_decline = 1;  // leave products with at most four channel pairs per block to the any-l forward kernel
int g_fwd_ti = 0;                    // 0 = widest tile that divides every n1, else force 1 / 2 / 4
int g_bwd_enable = 1;
int g_bwd_one_enable = 1; // the backward kernel for calls with one triple
int g_bwd_l6_split = 1;     // operands above l = 4, product above l = 6: two launches of the unrolled kernels (l <= 6, l >= 7)
int g_bwd_split = 1;        // backward launches with few cells deal the pairs of a cell to several blocks
int g_bwd_split_below = 1024;  // ... when the launch would have fewer blocks than this (four per compute unit)
int g_bwd_split_max = 16;   // ... to at most this many blocks per cell (headline type, 64 cells: 115 us with one block per cell, 43 with 8, 37 with 16, 51 with 25)
int g_bwd_one_wide = 1;   // ... and the one for a second operand of 16 or 32 channels (0 off, else cells per wave and block)
long long g_bwd_one_wide_cells = 4096;  // ... in launches with at least this many cells (a wave takes whole cells)
int g_bwd_l6_enable = 1;  // the backward kernel for operands up to l = 6
int g_bwd_min_runs = 128;           // runs of 64 slots a backward block should have at least, LDS allowing (0: no such rule)
int g_bwd_lds_target = 40 * 1024;  // LDS bytes per block the backward kernel aims at when it picks the cells per block
int g_fwd_enable = 1;
int g_fwd_l6_enable = 1;  // the forward kernel for operands up to l = 6

struct DevicePlan {
  std::vector<PairRec> pairs;
  PairRec *d_pairs = nullptr;
  float *d_bank = nullptr;
  int bank_len = 0;
  int zero_off = 0;  // a run of zeros in the bank (stand-in table and stand-in row for absent parts)
  bool padded = false;  // some channel count is not a power of two: the backward pass runs the padded kernels
  int xsize = 0, ysize = 0;
};

std::mutex g_plan_mutex;
std::map<std::vector<int>, DevicePlan> g_plans;  // key starts with the device ordinal

}  // namespace

// (b, g0, g1) -> one cell index with one stride, if the strides nest; broadcast-everywhere gives stride 0.
bool collapse(const PartDev &p, const long long E[3], const long long own[3], long long *cell_stride) {
  const long long s[3] = {p.sb, p.sg0, p.sg1};
  int dims[3], nd = 0;
  for (int d = 0; d < 3; d++)
    if (E[d] > 1) dims[nd++] = d;
  if (nd == 0) {
    *cell_stride = 0;
    return true;
  }
  bool all_bcast = true, none_bcast = true;
  for (int k = 0; k < nd; k++) {
    if (own[dims[k]] == E[dims[k]]) all_bcast = false;
    else none_bcast = false;
  }
  if (all_bcast) {
    *cell_stride = 0;
    return true;
  }
  if (!none_bcast) return false;
  for (int k = 0; k + 1 < nd; k++)
    if (s[dims[k]] != E[dims[k + 1]] * s[dims[k + 1]]) return false;
  *cell_stride = s[dims[nd - 1]];
  return true;
}

bool to_fast(const PartDev &p, const long long E[3], const long long own[3], int n, bool is_dest, FastPart *out) {
  if (n > 1 && p.sc != 1) return false;
  if (p.sm < 0 || p.sm > 0x3fffffffLL) return false;
  long long cs;
  if (!collapse(p, E, own, &cs)) return false;
  const long long cells = E[0] * E[1] * E[2];
  if (is_dest && cells > 1 && cs == 0) return false;  // a broadcast destination needs a reduction over cells
  out->ptr = p.ptr;
  out->sb = cs;
  out->sm = (int)p.sm;
  out->n = n;
  return true;
}

PartDev desc_to_dev(const gelib_part_desc *d, const long long E[3], long long own[3]) {
  PartDev p;
  p.ptr = (float2 *)d->ptr;
  long long s[3];
  for (int k = 0; k < 3; k++) {
    own[k] = (d->dims[k] == E[k]) ? E[k] : 1;
    s[k] = (d->dims[k] == E[k] && E[k] > 1) ? d->strides[k] : 0;
  }
  p.sb = s[0];
  p.sg0 = s[1];
  p.sg1 = s[2];
  p.sm = d->strides[3];
  p.sc = d->strides[4];
  return p;
}

bool is_pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }
int ilog2(int v) {
  int k = 0;
  while ((1 << k) < v) k++;
  return k;
}

namespace {

// Step records for the backward kernels: for every pair, the coefficients of its (m1,m2) steps in the order the kernel
// runs them (row number m = m1 + m2 rising from -ltop, m1 rising inside a row): C_l[m1,m2] for the l from
// max(|l1-l2|, lo, |m|) to ltop = min(l1+l2, cap), zero where the part is absent (rec_pos in cg_unrolled_bwd_impl.h is
// the same count on the device side).  cap is the largest l the kernel that will run has code for (unrolled_bwd_cap).
// A pair's records start on a 64-byte boundary of the device allocation and are padded to whole groups of 32 floats,
// the unit the kernel loads.
void append_step_records(bool diag, int cap, int lo, size_t pair_bytes, std::vector<PairRec> *pairs, std::vector<float> *bank) {
  (void)diag;
  for (auto &p : *pairs) p.rec_off = -1;
  if (cap < 0) return;
  while ((pair_bytes + bank->size() * sizeof(float)) % 64) bank->push_back(0.f);
  for (auto &p : *pairs) {
    const int lmin = std::max(std::abs(p.l1 - p.l2), lo), ltop = std::min(p.l1 + p.l2, cap);
    const int dl0 = lmin - std::abs(p.l1 - p.l2);   // the pair's tables are indexed from |l1 - l2|
    if (lmin > ltop) continue;
    const int nl = ltop - lmin + 1, w2 = 2 * p.l2 + 1;
    p.rec_off = (int)bank->size();
    // a step holds one coefficient for every l of the pair with a row m (l >= |m|), zero where the triple is absent
    for (int m = -ltop; m <= ltop; m++)
      for (int m1 = std::max(-p.l1, m - p.l2); m1 <= std::min(p.l1, m + p.l2); m1++) {
        const int m2 = m - m1;
        for (int dl = std::max(lmin, std::abs(m)) - lmin; dl < nl; dl++) {
          float c = 0.f;
          if (dl0 + dl < kMaxDl && p.ri[dl0 + dl] >= 0)
            c = (*bank)[p.cg_base + p.cg[dl0 + dl] + (m1 + p.l1) * w2 + (m2 + p.l2)];
          bank->push_back(c);
        }
      }
    while (bank->size() % 32) bank->push_back(0.f);  // the kernel fetches whole groups of 32 floats
  }
}

// Build (or fetch) the device tables for a list of triples.  xs/ys/rs give (l, n) of the l-sorted parts.
int get_plan(bool diag, const std::vector<VecTriple> &triples, const std::vector<std::pair<int, int>> &xs,
             const std::vector<std::pair<int, int>> &ys, const std::vector<int> &rls, const DevicePlan **out) {
  int dev = 0;
  GELIB_HIP_TRY(hipGetDevice(&dev));
  std::vector<int> key = {dev, diag ? 1 : 0, (int)xs.size(), (int)ys.size(), (int)rls.size()};
  for (auto &v : xs) key.push_back(v.first), key.push_back(v.second);
  for (auto &v : ys) key.push_back(v.first), key.push_back(v.second);
  for (int l : rls) key.push_back(l);
  for (auto &t : triples) key.push_back(t.ri), key.push_back(t.offs);
  // a PairRec has room for kMaxDl values of l per pair; callers decline wider products before they come here
  for (auto &t : triples)
    if (t.l - std::abs(t.l1 - t.l2) < 0 || t.l - std::abs(t.l1 - t.l2) >= kMaxDl) return GELIB_HIP_ERR_UNSUPPORTED;
  std::lock_guard<std::mutex> lock(g_plan_mutex);
  auto it = g_plans.find(key);
  if (it != g_plans.end()) {
    *out = &it->second;
    return GELIB_HIP_OK;
  }
  DevicePlan plan;
  std::vector<float> bank;
  std::vector<int> xoff(xs.size()), yoff(ys.size());
  for (size_t i = 0; i < xs.size(); i++) {
    xoff[i] = plan.xsize;
    plan.xsize += (2 * xs[i].first + 1) * xs[i].second;
  }
  for (size_t i = 0; i < ys.size(); i++) {
    yoff[i] = plan.ysize;
    plan.ysize += (2 * ys[i].first + 1) * ys[i].second;
  }
  for (auto &t : triples) {
    PairRec *p = nullptr;
    if (!plan.pairs.empty() && plan.pairs.back().xi == t.xi && plan.pairs.back().yi == t.yi) p = &plan.pairs.back();
    if (!p) {
      PairRec rec;
      std::memset(&rec, 0, sizeof(rec));
      rec.xi = t.xi;
      rec.yi = t.yi;
      rec.l1 = t.l1;
      rec.l2 = t.l2;
      rec.n1 = xs[t.xi].second;
      rec.n2 = ys[t.yi].second;
      for (int d = 0; d < kMaxDl; d++) rec.ri[d] = -1;
      rec.cg_base = (int)bank.size();
      {
        // lane slots: channel counts rounded up to powers of two (the backward lane sums need aligned groups);
        // slots beyond the real channels are idle lanes of the padded kernels
        const int lg1 = ilog2(std::max(1, rec.n1)), lg2 = ilog2(std::max(1, rec.n2));
        const int lgu = diag ? lg1 : lg1 + lg2;
        rec.lg_n2p = lg2;
        rec.log2_u = lgu <= 20 ? lgu : -1;
        rec.rpc = 0;
        rec.rpc_magic = 0;
        if (lgu >= 6 && lgu <= 20) {
          const long long pow2_slots = 1LL << lgu, tight = (long long)rec.n1 * (diag ? 1 : (1LL << lg2));
          rec.rpc = (int)((tight % 64 == 0 ? tight : pow2_slots) / 64);
          if (rec.rpc > 1) rec.rpc_magic = (unsigned)(((1ULL << 32) + rec.rpc - 1) / rec.rpc);
        }
        if (!is_pow2(rec.n1) || (!diag && !is_pow2(rec.n2))) plan.padded = true;
      }
      rec.xoff = xoff[t.xi];
      rec.yoff = yoff[t.yi];
      plan.pairs.push_back(rec);
      p = &plan.pairs.back();
    }
    const int dl = t.l - std::abs(t.l1 - t.l2);
    p->ri[dl] = t.ri;
    p->offs[dl] = t.offs;
    p->cg[dl] = (int)bank.size() - p->cg_base;
    const size_t n = (size_t)(2 * t.l1 + 1) * (2 * t.l2 + 1);
    bank.resize(bank.size() + n);
    cg_matrix_host(t.l1, t.l2, t.l, bank.data() + bank.size() - n);
    p->cg_len = (int)bank.size() - p->cg_base;
  }
  {
    // rank of every pair by falling cost (terms of its triples times lane slots): launches that deal the pairs of a
    // cell to S blocks give block s the pairs of rank s, s + S, ...
    std::vector<long long> cost(plan.pairs.size(), 0);
    for (auto &t : triples) {
      size_t k = 0;
      while (k < plan.pairs.size() && !(plan.pairs[k].xi == t.xi && plan.pairs[k].yi == t.yi)) k++;
      long long terms = 0;
      for (int m = -t.l; m <= t.l; m++) terms += std::min(t.l1, m + t.l2) - std::max(-t.l1, m - t.l2) + 1;
      cost[k] += terms * (diag ? plan.pairs[k].n1 : (long long)plan.pairs[k].n1 * plan.pairs[k].n2);
    }
    std::vector<int> order(plan.pairs.size());
    for (size_t k = 0; k < order.size(); k++) order[k] = (int)k;
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return cost[a] > cost[b]; });
    for (size_t r = 0; r < order.size(); r++) plan.pairs[order[r]].cost_rank = (int)r;
  }
  if (bank.size() % 2) bank.push_back(0.f);
  plan.zero_off = (int)bank.size();
  bank.resize(bank.size() + (2 * kLTMax + 1) * (2 * kLTMax + 1) + 1, 0.f);
  const size_t pair_bytes = plan.pairs.size() * sizeof(PairRec);
  {
    int lcap = 0, lop = 0, llo = 1 << 30;
    for (auto &t : triples) lcap = std::max(lcap, t.l), lop = std::max(lop, std::max(t.l1, t.l2)), llo = std::min(llo, t.l);
    append_step_records(diag, unrolled_bwd_cap(lcap, lop, llo), unrolled_bwd_lo(lcap, lop, llo), pair_bytes, &plan.pairs, &bank);
  }
  plan.bank_len = (int)bank.size();
  const size_t bank_bytes = bank.size() * sizeof(float);
  char *d = nullptr;
  GELIB_HIP_TRY(hipMalloc((void **)&d, pair_bytes + bank_bytes));
  hipError_t e = hipMemcpy(d, plan.pairs.data(), pair_bytes, hipMemcpyHostToDevice);
  if (e == hipSuccess) e = hipMemcpy(d + pair_bytes, bank.data(), bank_bytes, hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    (void)hipFree(d);
    return record_hip_error(e, "hipMemcpy(plan)");
  }
  plan.d_pairs = (PairRec *)d;
  plan.d_bank = (float *)(d + pair_bytes);
  auto ins = g_plans.emplace(key, std::move(plan));
  *out = &ins.first->second;
  return GELIB_HIP_OK;
}

struct FastLists {
  std::vector<FastPart> x, y, r, xg, yg;
};

int run_fwd(bool diag, const std::vector<VecTriple> &triples, const std::vector<std::pair<int, int>> &xs,
            const std::vector<std::pair<int, int>> &ys, const std::vector<int> &rls, const FastLists &f,
            long long ncells, int offs_add, bool accumulate, hipStream_t s, int *used) {
  *used = 0;
  // With at most four channel pairs per (l1,l2) block a store instruction of this kernel writes 32 bytes or less per
  // cell; the any-l forward kernel, whose lanes own whole output rows of a cell, does better there (L=4, measured in
  // one process: 2 channels 14.5 ms here, 9.3 ms there; 1 channel 23.3 / 12.2; from 4 channels on this kernel wins,
  // 5.8 / 8.8 ms).
  if (!diag && g_fwd_narrow_decline) {
    long long widest = 0;
    for (auto &t : triples) widest = std::max(widest, (long long)xs[t.xi].second * ys[t.yi].second);
    if (widest <= 4 && triples.size() > 1) return GELIB_HIP_OK;
  }
  // one cell's two operand parts must fit the LDS staging area
  for (auto &t : triples) {
    const long long op_bytes = 8LL * ((2 * t.l1 + 1) * (long long)xs[t.xi].second + (2 * t.l2 + 1) * (long long)ys[t.yi].second);
    if (op_bytes > g_fwd_lds_bytes) return GELIB_HIP_OK;
  }
  // which kernel would run is decided from the type alone, before any table is built: a product this family declines
  // (e.g. operands of l = 6 uncapped) must not cost a device allocation, and its l range does not fit a PairRec
  int ti = 1;
  if (!diag) {
    ti = 4;
    for (auto &t : triples) {
      const int n1 = xs[t.xi].second, n2 = ys[t.yi].second;
      while (ti > 1 && n1 % ti) ti >>= 1;
      // four channels of x per thread leave n1/4 * n2 slots per cell: with few channels the pieces one store
      // instruction writes per cell get too short (8 channels: 4.77 -> 4.34 ms, 4 channels: 8.3 -> 6.9 ms with two)
      if (n1 < 16 && ti > 2) ti = 2;
      // ... and so do few channels of the second operand (features x single-channel harmonics: 16 x 1 channels,
      // L=4 x L=2, B=1M 9.85 -> 8.5 ms; 32 x 1 channels 8.6 -> 7.5 ms)
      if (ti > 2 && (n1 / ti) * n2 < 16) ti = 2;
    }
    if (g_fwd_ti == 1 || g_fwd_ti == 2 || g_fwd_ti == 4) ti = std::min(ti, g_fwd_ti);
  }
  int lcap_all = 0, lop = 0;
  for (auto &t : triples) lcap_all = std::max(lcap_all, t.l), lop = std::max(lop, std::max(t.l1, t.l2));
  if (lop > kLT && ti == 4) ti = 2;  // the kernel for operands above kLT is built for two channels per thread
  if (!unrolled_fwd_takes(diag, ti, lcap_all, lop) || (lop > kLT && !g_fwd_l6_enable)) return GELIB_HIP_OK;
  const DevicePlan *plan = nullptr;
  int rc = get_plan(diag, triples, xs, ys, rls, &plan);
  if (rc) return rc;
  FwdArgs a;
  std::memset(&a, 0, sizeof(a));
  for (size_t i = 0; i < f.x.size(); i++) a.x[i] = f.x[i];
  for (size_t i = 0; i < f.y.size(); i++) a.y[i] = f.y[i];
  for (size_t i = 0; i < f.r.size(); i++) a.r[rls[i]] = f.r[i];  // indexed by l
  a.pairs = plan->d_pairs;
  a.bank = plan->d_bank;
  a.ncells = ncells;
  a.npairs = (int)plan->pairs.size();
  a.offs_add = offs_add;
  a.accumulate = accumulate ? 1 : 0;
  long long nblocks = 0;
  size_t lds_bytes = 0;
  int lcap = 0;
  for (auto &t : triples) lcap = std::max(lcap, t.l);
  // The cells are cut into tiles; the blocks of a tile (every pair, every run of cells inside the tile) have
  // consecutive indices, so blocks that run at the same time write into the same neighbourhood of every product part.
  // Measured in one process, forward pass: L=4 with 16 channels 4.41 ms at 64 cells per tile, 4.30 at 32, 4.56 at 128;
  // 8 channels 4.34 at 32 and 64, 4.89 at 4096; 4 channels (128-byte pieces per pair and row) 7.0 at 64, 6.7 at 1024,
  // 5.85 at 4096, 7.9 with all cells in one tile.
  long long auto_tile = 4096;
  for (auto &p : plan->pairs)
    if ((long long)p.n1 * (diag ? 1 : p.n2) >= 64) auto_tile = 32;
  const long long want_tile = g_fwd_cell_tile < 0 ? auto_tile : g_fwd_cell_tile;
  const long long tile = want_tile > 0 ? std::min<long long>(want_tile, ncells) : ncells;
  // product bytes a block aims at: 96 KB; 128 KB for products that reach above l = 4 (measured in one process on L=4,
  // 16 channels, 32768 cells: capped at l = 4 4.32 ms at 96 KB, 5.19 at 64 KB, 4.89 at 128 KB; uncapped 7.78 ms at
  // 96 KB, 8.12 at 64 KB, 7.42 at 128 KB)
  const long long block_bytes = g_fwd_block_bytes > 0 ? g_fwd_block_bytes : (lcap > kLT ? 128 * 1024 : 96 * 1024);
  for (int i = 0; i < a.npairs; i++) {
    const PairRec &p = plan->pairs[i];
    long long rows = 0;
    for (int d = 0; d < kMaxDl; d++)
      if (p.ri[d] >= 0) rows += 2 * (std::abs(p.l1 - p.l2) + d) + 1;
    const long long nout = diag ? p.n1 : (long long)p.n1 * p.n2;
    const long long bytes_per_cell = rows * nout * 8;
    const long long U = diag ? p.n1 : (long long)(p.n1 / ti) * p.n2;
    long long cpb = std::max<long long>(1, block_bytes / std::max<long long>(1, bytes_per_cell));
    const long long op_bytes = 8LL * ((2 * p.l1 + 1) * (long long)p.n1 + (2 * p.l2 + 1) * (long long)p.n2);
    cpb = std::min(cpb, std::max<long long>(1, g_fwd_lds_bytes / op_bytes));
    cpb = std::min<long long>(cpb, std::max<long long>(1, (1LL << 28) / std::max<long long>(1, U)));
    cpb = std::min(cpb, tile);
    cpb = (tile + (tile + cpb - 1) / cpb - 1) / ((tile + cpb - 1) / cpb);  // equal shares of the tile, not a short last block
    a.cpb[i] = (int)cpb;
    lds_bytes = std::max(lds_bytes, (size_t)(cpb * op_bytes));
    a.first_block[i] = (int)nblocks;
    nblocks += (tile + cpb - 1) / cpb;
    if (nblocks > 0x7fffffffLL) return GELIB_HIP_ERR_ARG;
  }
  a.first_block[a.npairs] = (int)nblocks;  // blocks of one tile
  a.tile = tile;
  a.blocks_per_tile = (int)nblocks;
  nblocks *= (ncells + tile - 1) / tile;
  if (nblocks > 0x7fffffffLL) return GELIB_HIP_ERR_ARG;
  rc = launch_unrolled_fwd(a, diag, ti, lcap, lop, (int)nblocks, lds_bytes, s);
  if (rc) return rc;
  *used = 1;
  return GELIB_HIP_OK;
}

int run_bwd(bool diag, const std::vector<VecTriple> &triples, const std::vector<std::pair<int, int>> &xs,
            const std::vector<std::pair<int, int>> &ys, const std::vector<int> &rls, const FastLists &f,
            long long ncells, int offs_add, bool accumulate, bool want_x, bool want_y, hipStream_t s, int *used) {
  *used = 0;
  int lcap = 0, lop = 0, llo = 1 << 30;
  bool padded = false;
  for (auto &t : triples) {
    lcap = std::max(lcap, t.l);
    llo = std::min(llo, t.l);
    lop = std::max(lop, std::max(t.l1, t.l2));
    padded = padded || !is_pow2(xs[t.xi].second) || (!diag && !is_pow2(ys[t.yi].second));
  }
  if (!unrolled_bwd_takes(diag, padded, lcap, lop, llo) || (lop > kLT && !g_bwd_l6_enable)) return GELIB_HIP_OK;
  // lane slots are the channel counts rounded up to powers of two; the reduced operand must fit a wave
  int u_min = 1 << 30;
  for (auto &t : triples) {
    const int n1 = xs[t.xi].second, n2 = ys[t.yi].second;
    if (n1 < 1 || n2 < 1) return GELIB_HIP_OK;
    const int lg1 = ilog2(n1), lg2 = ilog2(n2);
    if (!diag && lg2 > 8) return GELIB_HIP_OK;
    const int lgu = diag ? lg1 : lg1 + lg2;
    if (lgu > 20) return GELIB_HIP_OK;
    u_min = std::min<int>(u_min, 1 << lgu);
  }
  const DevicePlan *plan = nullptr;
  int rc = get_plan(diag, triples, xs, ys, rls, &plan);
  if (rc) return rc;
  BwdArgs a;
  std::memset(&a, 0, sizeof(a));
  for (size_t i = 0; i < f.x.size(); i++) a.x[i] = f.x[i];
  for (size_t i = 0; i < f.y.size(); i++) a.y[i] = f.y[i];
  for (size_t i = 0; i < f.r.size(); i++) a.g[rls[i]] = f.r[i];  // indexed by l
  for (size_t i = 0; i < f.xg.size(); i++) a.xg[i] = f.xg[i];
  for (size_t i = 0; i < f.yg.size(); i++) a.yg[i] = f.yg[i];
  a.pairs = plan->d_pairs;
  a.bank = plan->d_bank;
  a.ncells = ncells;
  a.npairs = (int)plan->pairs.size();
  a.nx = (int)xs.size();
  a.ny = (int)ys.size();
  a.offs_add = offs_add;
  a.accumulate = accumulate ? 1 : 0;
  a.want_x = want_x ? 1 : 0;
  a.want_y = want_y ? 1 : 0;
  a.bank_len = plan->bank_len;
  a.zero_off = plan->zero_off;
  a.padded = plan->padded ? 1 : 0;
  a.xsize = plan->xsize;
  a.ysize = plan->ysize;
  for (size_t i = 0; i < xs.size(); i++) a.xrows[i] = 2 * xs[i].first + 1;
  for (size_t i = 0; i < ys.size(); i++) a.yrows[i] = 2 * ys[i].first + 1;
  // enough cells per block to give every wave a full run of 64 slots, as far as LDS allows
  int cpb = std::max(1, kBlock / std::min(kBlock, u_min));
  // ... but no more than leave LDS for the blocks the registers allow on a compute unit (four; three for the kernel
  // for operands above kLT), as long as the block keeps at least two runs per wave; 64 KB at most in any case
  const size_t lds_target = lop > kLT ? 52 * 1024 : (size_t)g_bwd_lds_target;
  auto runs_at = [&](int c) {
    long long runs = 0;
    for (auto &p : plan->pairs) runs += p.rpc > 0 ? (long long)c * p.rpc : (((long long)c << p.log2_u) + kWave - 1) / kWave;
    return runs;
  };
  // few runs per cell (few pairs, few channels): more cells per block, so that the staging of the operands, the two
  // barriers and the write-out of a block are shared by at least g_bwd_min_runs runs
  // (as long as the launch keeps eight blocks per compute unit)
  while (g_bwd_min_runs > 0 && runs_at(cpb) < g_bwd_min_runs && cpb < 64 && ncells / (2 * cpb) >= 2048 &&
         unrolled_bwd_lds_bytes(a.bank_len, a.xsize, a.ysize, 2 * cpb) <= lds_target)
    cpb <<= 1;
  while (cpb > 1) {
    const size_t need = unrolled_bwd_lds_bytes(a.bank_len, a.xsize, a.ysize, cpb);
    if (need <= lds_target) break;
    if (need <= 64 * 1024 && runs_at(cpb / 2) < 2 * (kBlock / kWave)) break;
    cpb >>= 1;
  }
  const size_t lds = unrolled_bwd_lds_bytes(a.bank_len, a.xsize, a.ysize, cpb);
  if (lds > 150 * 1024) return GELIB_HIP_OK;
  a.cells_per_block = cpb;
  a.only_dl = -1;
  if (triples.size() == 1 && !diag && !plan->padded && lop <= kLT && g_bwd_one_enable)
    a.only_dl = triples[0].l - std::abs(triples[0].l1 - triples[0].l2);
  if (a.only_dl >= 0 && g_bwd_one_wide > 0) {
    const int n1 = xs[triples[0].xi].second, n2 = ys[triples[0].yi].second;
    // every wave of that kernel takes whole cells: it needs launches with cells enough to fill the GPU that way
    if ((n2 == 16 || n2 == 32) && n1 >= 16 && is_pow2(n1) && ncells >= g_bwd_one_wide_cells) {
      const int cpb1 = 4 * std::max(1, g_bwd_one_wide);
      a.cells_per_block = cpb1;
      const long long nb = (ncells + cpb1 - 1) / cpb1;
      if (nb > 0x7fffffffLL) return GELIB_HIP_ERR_ARG;
      rc = launch_one_triple_bwd(a, n2 / 16, triples[0].l1, triples[0].l2, triples[0].l, (int)nb,
                                 one_triple_bwd_lds_bytes(a.xsize, a.ysize), s);
      if (rc) return rc;
      *used = 1;
      return GELIB_HIP_OK;
    }
  }
  const long long nblocks = (ncells + cpb - 1) / cpb;
  if (nblocks > 0x7fffffffLL) return GELIB_HIP_ERR_ARG;
  a.pair_split = 1;
  // Few cells: a block would walk through all pairs of its cells while most of the GPU idles (L=4, 16 channels, 64
  // cells: 64 blocks of 25 pairs each, 111 us).  The pairs of a cell are then dealt to several blocks, whose partial
  // sums a second small kernel adds in a fixed order.
  if (g_bwd_split && a.only_dl < 0 && a.npairs > 1 && nblocks < g_bwd_split_below) {
    long long S = std::min<long long>({(long long)g_bwd_split_max, 32LL /* most blocks per cell the summing kernel adds */, (long long)a.npairs,
                                      (g_bwd_split_below + nblocks - 1) / nblocks});
    if (S >= 2) {
      const size_t xbytes = want_x ? sizeof(float2) * (size_t)S * ncells * a.xsize : 0;
      const size_t ybytes = want_y ? sizeof(float2) * (size_t)S * ncells * a.ysize : 0;
      std::lock_guard<std::mutex> lock(stream_scratch_mutex(1));
      void *buf = nullptr;
      if ((rc = stream_scratch(1, s, xbytes + ybytes, &buf))) return rc;
      if (buf) {  // none while the call is recorded into a graph: one block per cell then
        a.pair_split = (int)S;
        a.part_x = (float2 *)buf;
        a.part_y = (float2 *)((char *)buf + xbytes);
        if ((rc = launch_unrolled_bwd(a, diag, lcap, lop, (int)(nblocks * S), lds, s))) return rc;
        if ((rc = launch_unrolled_bwd_sum_splits(a, (int)nblocks, s))) return rc;
        *used = 1;
        return GELIB_HIP_OK;
      }
    }
  }
  rc = launch_unrolled_bwd(a, diag, lcap, lop, (int)nblocks, lds, s);
  if (rc) return rc;
  *used = 1;
  return GELIB_HIP_OK;
}

}  // namespace

int unrolled_part(int kind, const PartOp &op, bool accumulate, hipStream_t s, int *used) {
  *used = 0;
  if (op.l1 > kLTMax || op.l2 > kLTMax) return GELIB_HIP_OK;  // (above kLT: run_fwd / run_bwd say what they take)
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
  if (kind == 0) {
    return run_fwd(op.diag, triples, xs, ys, rls, f, ncells, op.offs, accumulate, s, used);
  }
  if (kind == 1) f.xg = f.x;  // destination
  if (kind == 2) f.yg = f.y;
  return run_bwd(op.diag, triples, xs, ys, rls, f, ncells, op.offs, accumulate, kind == 1, kind == 2, s, used);
}

bool lists_to_fast(const std::vector<const gelib_part_desc *> &ds, const long long E[3], bool is_dest,
                   std::vector<FastPart> *out, std::vector<std::pair<int, int>> *ln) {
  out->resize(ds.size());
  for (size_t i = 0; i < ds.size(); i++) {
    long long own[3];
    PartDev p = desc_to_dev(ds[i], E, own);
    const int l = (int)(ds[i]->dims[3] - 1) / 2, n = (int)ds[i]->dims[4];
    if (!to_fast(p, E, own, n, is_dest, &(*out)[i])) return false;
    if (ln) ln->push_back({l, n});
  }
  return true;
}

int unrolled_vec_fwd(const VecPlan &plan, const std::vector<const gelib_part_desc *> &r,
                     const std::vector<const gelib_part_desc *> &x, const std::vector<const gelib_part_desc *> &y,
                     bool accumulate, hipStream_t s, int *used) {
  *used = 0;
  if (!g_fwd_enable) return GELIB_HIP_OK;
  if (x.size() > (size_t)kFastIn || y.size() > (size_t)kFastIn || r.size() > (size_t)kFastOut) return GELIB_HIP_OK;
  for (auto *d : x)
    if ((d->dims[3] - 1) / 2 > kLTMax) return GELIB_HIP_OK;
  for (auto *d : y)
    if ((d->dims[3] - 1) / 2 > kLTMax) return GELIB_HIP_OK;
  for (auto *d : r)
    if ((d->dims[3] - 1) / 2 > 2 * kLTMax) return GELIB_HIP_OK;
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

int unrolled_vec_bwd(const VecPlan &plan, const std::vector<const gelib_part_desc *> &g,
                     const std::vector<const gelib_part_desc *> &x, const std::vector<const gelib_part_desc *> &y,
                     const std::vector<const gelib_part_desc *> &xg, const std::vector<const gelib_part_desc *> &yg,
                     bool accumulate, hipStream_t s, int *used) {
  *used = 0;
  if (!g_bwd_enable) return GELIB_HIP_OK;
  if (x.size() > (size_t)kFastIn || y.size() > (size_t)kFastIn || g.size() > (size_t)kFastOut) return GELIB_HIP_OK;
  for (auto *d : x)
    if ((d->dims[3] - 1) / 2 > kLTMax) return GELIB_HIP_OK;
  for (auto *d : y)
    if ((d->dims[3] - 1) / 2 > kLTMax) return GELIB_HIP_OK;
  for (auto *d : g)
    if ((d->dims[3] - 1) / 2 > 2 * kLTMax) return GELIB_HIP_OK;
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
  // A CGproduct of operands above l = 4 that reaches above l = 6 (the API default is uncapped): the triples up to l = 6
  // run on the kernel built for them, the rest on the one built for l = 7..12, which adds onto what the first wrote.
  // Each launch reads its own parts of g, so g is still read once.
  {
    int lcap = 0, lop = 0, llo = 1 << 30;
    bool padded = false;
    for (auto &t : plan.triples) {
      lcap = std::max(lcap, t.l), llo = std::min(llo, t.l), lop = std::max(lop, std::max(t.l1, t.l2));
      padded = padded || !is_pow2(xs[t.xi].second) || !is_pow2(ys[t.yi].second);
    }
    // (one pair of parts with channel counts that are not powers of two is left to the single-pair kernels: (5, 3
    // channels) x (6, 5 channels), 65536 cells: 2.4 ms here with padded lane slots, 1.2 ms there)
    const bool one_padded_pair = padded && xs.size() == 1 && ys.size() == 1;
    if (!plan.diag && !one_padded_pair && g_bwd_l6_enable && g_bwd_l6_split && lop > kLT && lop <= kLTMax && llo <= kLTMax &&
        lcap > kLTMax && lcap <= 2 * kLTMax) {
      std::vector<VecTriple> ta, tb;
      std::vector<int> rla, rlb, map_a(rls.size(), -1), map_b(rls.size(), -1);
      FastLists fa = f, fb = f;
      fa.r.clear();
      fb.r.clear();
      for (size_t k = 0; k < rls.size(); k++) {
        if (rls[k] <= kLTMax) map_a[k] = (int)rla.size(), rla.push_back(rls[k]), fa.r.push_back(f.r[k]);
        else map_b[k] = (int)rlb.size(), rlb.push_back(rls[k]), fb.r.push_back(f.r[k]);
      }
      for (auto t : plan.triples) {
        if (t.l <= kLTMax) t.ri = map_a[t.ri], ta.push_back(t);
        else t.ri = map_b[t.ri], tb.push_back(t);
      }
      int rc = run_bwd(false, ta, xs, ys, rla, fa, ncells, 0, accumulate, !xg.empty(), !yg.empty(), s, used);
      if (rc || !*used) return rc;
      int used_b = 0;
      rc = run_bwd(false, tb, xs, ys, rlb, fb, ncells, 0, true, !xg.empty(), !yg.empty(), s, &used_b);
      if (rc) return rc;
      return used_b ? GELIB_HIP_OK : GELIB_HIP_ERR_ARG;   // the same operands and cells: what took the first part takes the second
    }
  }
  return run_bwd(plan.diag, plan.triples, xs, ys, rls, f, ncells, 0, accumulate, !xg.empty(), !yg.empty(), s, used);
}

int unrolled_set_option(const char *name, int value) {
  if (!std::strcmp(name, "fwd_block_bytes")) {
    if (value != 0 && value < 1024) return GELIB_HIP_ERR_ARG;
    g_fwd_block_bytes = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "fwd_lds_bytes")) {
    if (value < 1024 || value > 60 * 1024) return GELIB_HIP_ERR_ARG;
    g_fwd_lds_bytes = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "fwd_cell_tile")) {
    if (value < -1) return GELIB_HIP_ERR_ARG;
    g_fwd_cell_tile = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "fwd_narrow_decline")) {
    g_fwd_narrow_decline = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "fwd_tile")) {
    g_fwd_ti = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "unrolled_fwd")) {
    g_fwd_enable = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "bwd_min_runs")) {
    if (value < 0) return GELIB_HIP_ERR_ARG;
    g_bwd_min_runs = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "bwd_lds_target")) {
    if (value < 1024 || value > 150 * 1024) return GELIB_HIP_ERR_ARG;
    g_bwd_lds_target = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "unrolled_fwd_l6")) {
    g_fwd_l6_enable = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "unrolled_bwd_l6_split")) {
    g_bwd_l6_split = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "unrolled_bwd_split")) {
    g_bwd_split = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "unrolled_bwd_split_below")) {
    g_bwd_split_below = value > 0 ? value : 1024;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "unrolled_bwd_split_max")) {
    g_bwd_split_max = value > 1 ? value : 16;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "unrolled_bwd_one_wide_cells")) {
    g_bwd_one_wide_cells = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "unrolled_bwd_one_wide")) {  // 0 off, otherwise the cells per wave of a block of that kernel
    g_bwd_one_wide = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "unrolled_bwd_one")) {
    g_bwd_one_enable = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "unrolled_bwd_l6")) {
    g_bwd_l6_enable = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "unrolled_bwd")) {
    g_bwd_enable = value;
    return GELIB_HIP_OK;
  }
  return GELIB_HIP_ERR_ARG;
}

}  // namespace gelib_hip
