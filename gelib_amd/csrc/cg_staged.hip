// Forward and backward CG / DiagCG product for any l, with run-time m-loops; every triple of the product in one
// launch.
//
// A block owns a few whole cells and stages their operands x, y in LDS once.  The flattened (cell, channel slot)
// space of each triple is cut into runs of 64 slots and the block's waves take the runs of all triples in turn
// (round robin over one running count, so triples with a single run still spread over all waves).  A lane owns
// one channel pair (i, j) of the triple's block.
//
//   forward   for every output row m the lane sums C x[m1,i] y[m-m1,j] over m1 in a register and stores the row:
//             two LDS reads and six arithmetic instructions per term, stores contiguous across the wave.
//   backward  the lane first reads its 2l+1 values of g into registers (the only pass over g), then forms
//                 xg[m1,i] += sum_m2 C g[m1+m2] conj(y[m2,j])      yg[m2,j] += sum_m1 C g[m1+m2] conj(x[m1,i])
//             as two loop nests, each with a register accumulator for its inner sum.  The row of g is picked by a
//             run-time index that is the same for the whole wave, which the hardware supports directly
//             (register-relative addressing), so g needs no LDS; when 2l+1 exceeds the 16 or 32 rows a lane
//             keeps, g goes through the registers in windows and each window adds its share of the terms.  The inner sums are reduced over the lanes that
//             share i (resp. j) and added to the block's gradient images in LDS with LDS float atomics: several
//             waves add to one image, so the order of those additions is not fixed from run to run.  After the
//             last triple the images are written out in contiguous rows.
//
// The kernel arguments hold every part descriptor; the kernels read them through the kernel-argument pointer
// with run-time indices (scalar loads), never through the by-value parameter, which the compiler would copy to
// scratch memory as soon as one index is not a compile-time constant.
#include "cg_lane_sums.h"
#include "cg_staged.h"
#include "cg_unrolled_dev.h"

namespace gelib_hip {

namespace {

typedef float v2f __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v32f __attribute__((ext_vector_type(32)));
typedef __attribute__((address_space(1))) v2f GlobalC;   // complex number in global memory
typedef __attribute__((address_space(3))) float LdsF;    // float in LDS
typedef const __attribute__((address_space(3))) v2f *LdsC;  // complex numbers in LDS (32-bit address arithmetic)
typedef const __attribute__((address_space(4))) float *CoeffPtr;
typedef const __attribute__((address_space(4))) StagedTriple *TriplePtr;
typedef const __attribute__((address_space(4))) StagedArgs *ArgPtr;
typedef const __attribute__((address_space(4))) FastPart *PartPtr;
typedef const __attribute__((address_space(4))) int *IntPtr;

__device__ __forceinline__ ArgPtr kernel_args() { return (ArgPtr)__builtin_amdgcn_kernarg_segment_ptr(); }

__device__ __forceinline__ FastPart load_part(PartPtr p) {
  FastPart r;
  r.ptr = p->ptr;
  r.sb = p->sb;
  r.sm = p->sm;
  r.n = p->n;
  return r;
}

// Copies between memory and the packed per-cell LDS image of a part list (each part's rows contiguous).
// MODE 0: stage operands into LDS.  MODE 1: write the image out.  MODE 2: add the image to what is there.
template <int MODE>
__device__ __forceinline__ void copy_image(PartPtr parts, IntPtr rows, int nparts, float2 *img, int img_size,
                                           long long cell0, int ncell) {
  int off = 0;
  for (int k = 0; k < nparts; k++) {
    const FastPart P = load_part(parts + k);
    const int per_cell = rows[k] * P.n;
    const bool packed = P.sm == P.n;
    for (int c = 0; c < ncell; c++) {
      GlobalC *base = (GlobalC *)P.ptr + (cell0 + c) * P.sb;
      float2 *li = img + c * img_size + off;
      for (int r = threadIdx.x; r < per_cell; r += blockDim.x) {
        long long src = r;
        if (!packed) {
          const int m = r / P.n;
          src = (long long)m * P.sm + (r - m * P.n);
        }
        if (MODE == 0) {
          const v2f t = base[src];
          li[r] = make_float2(t.x, t.y);
        } else {
          const float2 v = li[r];
          v2f o = {v.x, v.y};
          if (MODE == 2) o += base[src];
          base[src] = o;
        }
      }
    }
    off += per_cell;
  }
}

// Which runs of the triple this wave takes: runs are numbered on across triples and dealt out round robin.
// base = (runs of all earlier triples) mod W on entry, updated on exit; returns the wave's first run.
__device__ __forceinline__ int first_run(int &base, int wave, int W, int nruns) {
  int first = wave - base;
  if (first < 0) first += W;
  base = (base + nruns) % W;
  return first;
}

// The coefficients of a loop nest form one stream of floats.  A wave keeps 128 consecutive entries of it spread over
// the lanes of two registers (lane k of `cur` holds entry base+k, of `nxt` entry base+64+k) and hands one entry at
// a time to the whole wave with a lane read, so the inner loops wait on no memory for their coefficients; the
// following 64 entries are requested a full register ahead of their use.
struct CoeffStream {
  const __attribute__((address_space(1))) float *src;
  int base;
  float cur, nxt;
  __device__ __forceinline__ void start(const float *bank, int pos, int lane) {
    src = (const __attribute__((address_space(1))) float *)bank;
    base = pos;
    cur = src[pos + lane];
    nxt = src[pos + kWave + lane];
  }
  // afterwards base <= pos < base + 64
  __device__ __forceinline__ void seek(int pos, int lane) {
    if (pos >= base + 2 * kWave) {  // a long skip: start over at pos
      base = pos;
      cur = src[pos + lane];
      nxt = src[pos + kWave + lane];
    } else if (pos >= base + kWave) {
      cur = nxt;
      base += kWave;
      nxt = src[base + kWave + lane];
    }
  }
};

__device__ __forceinline__ float lane_value(float v, int k) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), k));
}

// term(c) for the len <= 64 stream entries from pos on
template <class F>
__device__ __forceinline__ void for_coeffs(CoeffStream &cs, int pos, int len, int lane, F &&term) {
  cs.seek(pos, lane);
  // the position in the stream is the same for the whole wave; saying so keeps the loop counters scalar
  const int k = __builtin_amdgcn_readfirstlane(pos - cs.base);
  len = __builtin_amdgcn_readfirstlane(len);
  const int first = min(len, kWave - k);
  // four terms per trip: their LDS reads are independent, so the wave waits once for four of them
  int t = 0;
  for (; t + 4 <= first; t += 4) {
    const float c0 = lane_value(cs.cur, k + t), c1 = lane_value(cs.cur, k + t + 1);
    const float c2 = lane_value(cs.cur, k + t + 2), c3 = lane_value(cs.cur, k + t + 3);
    term(c0);
    term(c1);
    term(c2);
    term(c3);
  }
  for (; t < first; t++) term(lane_value(cs.cur, k + t));
  for (; t < len; t++) term(lane_value(cs.nxt, t - first));
}

// The same over a coefficient stream held in LDS (every lane reads the same address)
typedef const __attribute__((address_space(3))) float *LdsCoeffs;
template <class F>
__device__ __forceinline__ void for_coeffs_lds(LdsCoeffs c, int len, F &&term) {
  int t = 0;
  for (; t + 4 <= len; t += 4) {
    const float c0 = c[t], c1 = c[t + 1], c2 = c[t + 2], c3 = c[t + 3];
    term(c0);
    term(c1);
    term(c2);
    term(c3);
  }
  for (; t < len; t++) term(c[t]);
}

// ---- forward ------------------------------------------------------------------------------------------------------
typedef float v4f __attribute__((ext_vector_type(4)));

// TILE adjacent complex numbers from LDS / to global memory as 16-byte accesses
template <int TILE>
struct CTile {
  v2f v[TILE];
};

template <int TILE>
__device__ __forceinline__ CTile<TILE> lds_tile(LdsC p) {
  CTile<TILE> t;
  if constexpr (TILE == 1) {
    t.v[0] = *p;
  } else {
    static_for<TILE / 2>([&](auto hc) __attribute__((always_inline)) {
      constexpr int h = decltype(hc)::value;
      const v4f q = ((const __attribute__((address_space(3))) v4f *)p)[h];
      t.v[2 * h] = v2f{q.x, q.y};
      t.v[2 * h + 1] = v2f{q.z, q.w};
    });
  }
  return t;
}

template <int TILE>
__device__ __forceinline__ void store_tile(GlobalC *dst, const CTile<TILE> &t, bool accumulate) {
  if constexpr (TILE == 1) {
    v2f o = t.v[0];
    if (accumulate) o += *dst;
    *dst = o;
  } else {
    static_for<TILE / 2>([&](auto hc) __attribute__((always_inline)) {
      constexpr int h = decltype(hc)::value;
      __attribute__((address_space(1))) v4f *d4 = (__attribute__((address_space(1))) v4f *)dst + h;
      v4f o = {t.v[2 * h].x, t.v[2 * h].y, t.v[2 * h + 1].x, t.v[2 * h + 1].y};
      if (accumulate) o += *d4;
      *d4 = o;
    });
  }
}

// A lane owns TILE adjacent output channels (the same i and TILE adjacent j; for Diag TILE adjacent channels), so
// the per-row and per-term bookkeeping -- which is most of the instructions when rows are short -- is shared by
// TILE complex products.  The host picks TILE (1, 2 or 4) so that every channel count and offset is a multiple of
// it and the output pointers are 8*TILE-byte aligned.
// LDSC: the coefficient stream has been staged in LDS (it fits); otherwise it is streamed through lane reads.
template <bool DIAG, int TILE, bool LDSC>
__global__ void __launch_bounds__(1024) staged_fwd_kernel(const StagedArgs) {
  const ArgPtr a = kernel_args();
  extern __shared__ float2 staged_lds[];
  const int cpb = a->cpb, xsize = a->xsize, ysize = a->ysize;
  float2 *xs = staged_lds;
  float2 *ys = xs + cpb * xsize;
  const long long cell0 = (long long)blockIdx.x * cpb;
  const long long left = a->ncells - cell0;
  const int ncell = left < cpb ? (int)left : cpb;
  copy_image<0>(a->x, a->xrows, a->nx, xs, xsize, cell0, ncell);
  copy_image<0>(a->y, a->yrows, a->ny, ys, ysize, cell0, ncell);
  const float *bank = a->bank;
  float *coeffs = reinterpret_cast<float *>(ys + cpb * ysize);
  if (LDSC) {
    const int n = a->lds_coeffs;
    for (int e = threadIdx.x; e < n; e += blockDim.x) coeffs[e] = ((const __attribute__((address_space(1))) float *)bank)[e];
  }
  __syncthreads();

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & (kWave - 1);
  const int W = blockDim.x >> 6;
  const TriplePtr triples = (TriplePtr)a->triples;
  const int ntriples = a->ntriples, offs_add = a->offs_add;
  const bool accumulate = a->accumulate != 0;
  int base = 0;
  for (int t = 0; t < ntriples; t++) {
    const TriplePtr tr = triples + t;
    const int U = tr->u / TILE;  // tile slots per cell
    const int nruns = (cpb * U + kWave - 1) >> 6;
    const int first = first_run(base, wave, W, nruns);
    if (first >= nruns) continue;
    const int l1 = tr->l1, l2 = tr->l2, l = tr->l, n1 = tr->n1, n2 = tr->n2;
    const FastPart R = load_part(a->r + tr->ri);
    for (int run = first; run < nruns; run += W) {
      const int flat = (run << 6) + lane;
      const bool live = flat < ncell * U;
      const int fc = live ? flat : 0;  // dead lanes compute on valid data and never store
      const int cl = fc / U;
      const int u = (fc - cl * U) * TILE;
      const int i = DIAG ? u : u / n2;
      const int j = DIAG ? u : u - i * n2;
      const LdsC xb = (LdsC)xs + (cl * xsize + tr->xoff + i);
      const LdsC yb = (LdsC)ys + (cl * ysize + tr->yoff + j);
      GlobalC *rp = (GlobalC *)R.ptr + (cell0 + cl) * R.sb + (tr->offs + offs_add + u);
      int pos = tr->cg_fwd;
      CoeffStream cs;
      if (!LDSC) cs.start(bank, pos, lane);
      for (int m = -l; m <= l; m++) {
        const int m1lo = max(-l1, m - l2), m1hi = min(l1, m + l2);
        LdsC xp = xb + (m1lo + l1) * n1;
        LdsC yp = yb + (m - m1lo + l2) * n2;
        CTile<TILE> acc;
#pragma unroll
        for (int k = 0; k < TILE; k++) acc.v[k] = v2f{0.f, 0.f};
        auto term = [&](float c) __attribute__((always_inline)) {
          const CTile<DIAG ? TILE : 1> xt = lds_tile<DIAG ? TILE : 1>(xp);
          const CTile<TILE> yt = lds_tile<TILE>(yp);
          xp += n1;
          yp -= n2;
#pragma unroll
          for (int k = 0; k < TILE; k++) {
            const v2f xv = xt.v[DIAG ? k : 0], yv = yt.v[k];
            const float pr = c * xv.x, pi = c * xv.y;  // (C x) y, the reference's order
            acc.v[k].x = fmaf(pr, yv.x, acc.v[k].x);
            acc.v[k].x = fmaf(-pi, yv.y, acc.v[k].x);
            acc.v[k].y = fmaf(pr, yv.y, acc.v[k].y);
            acc.v[k].y = fmaf(pi, yv.x, acc.v[k].y);
          }
        };
        if (LDSC) for_coeffs_lds((LdsCoeffs)coeffs + pos, m1hi - m1lo + 1, term);
        else for_coeffs(cs, pos, m1hi - m1lo + 1, lane, term);
        pos += m1hi - m1lo + 1;
        if (live) store_tile<TILE>(rp + (long long)(m + l) * R.sm, acc, accumulate);
      }
    }
  }
}

// ---- backward -----------------------------------------------------------------------------------------------------
// The rows of g one lane holds, indexable with a wave-uniform run-time row number.
template <int CAP>
struct RowRegs;

template <>
struct RowRegs<16> {
  v16f re, im;
  __device__ __forceinline__ void clear() { re = 0.f, im = 0.f; }
  template <int M>
  __device__ __forceinline__ void set(float r, float i) {
    re[M] = r, im[M] = i;
  }
  __device__ __forceinline__ void get(int m, float &r, float &i) const { r = re[m], i = im[m]; }
  __device__ __forceinline__ void add(int m, float r, float i) { re[m] += r, im[m] += i; }
  template <int M>
  __device__ __forceinline__ float2 row() const {
    return make_float2(re[M], im[M]);
  }
};

template <>
struct RowRegs<32> {
  v32f re, im;
  __device__ __forceinline__ void clear() { re = 0.f, im = 0.f; }
  template <int M>
  __device__ __forceinline__ void set(float r, float i) {
    re[M] = r, im[M] = i;
  }
  __device__ __forceinline__ void get(int m, float &r, float &i) const { r = re[m], i = im[m]; }
  __device__ __forceinline__ void add(int m, float r, float i) { re[m] += r, im[m] += i; }
  template <int M>
  __device__ __forceinline__ float2 row() const {
    return make_float2(re[M], im[M]);
  }
};

template <int CAP>
constexpr int bwd_max_threads() {
  return CAP == 16 ? 1024 : 512;
}

// Rows w0 .. w0+CAP-1 of a lane's column of g into the registers.  Rows past the end repeat the last one (never
// used): the loads stay unconditional, which keeps the register rows one straight chain of writes instead of a
// merge of alternatives at every row.
// keep == false (a lane beyond the real channels) stores zeros.
template <int CAP>
__device__ __forceinline__ void load_window(RowRegs<CAP> &G, GlobalC *gp, int sm, int w0, int rows, bool keep) {
  static_for<CAP>([&](auto mc) __attribute__((always_inline)) {
    constexpr int M = decltype(mc)::value;
    const int row = min(w0 + M, rows - 1);
    const v2f v = gp[(long long)row * sm];
    G.template set<M>(keep ? v.x : 0.f, keep ? v.y : 0.f);
  });
}

// A backward lane's channel pair.  Lane slots are laid out n1p x n2p with the channel counts rounded up to powers
// of two, so that the lanes sharing i (resp. j) form aligned groups; a slot beyond the real channels reads channel 0,
// has its g forced to zero and never writes.
struct LaneChan {
  int i, j, chan;
  bool valid;
};
template <bool DIAG>
__device__ __forceinline__ LaneChan lane_chan(int u, int lg_n2p, int n1, int n2) {
  LaneChan c;
  c.i = DIAG ? u : (u >> lg_n2p);
  c.j = DIAG ? u : (u & ((1 << lg_n2p) - 1));
  c.valid = c.i < n1 && (DIAG || c.j < n2);
  if (!c.valid) c.i = 0, c.j = 0;
  c.chan = DIAG ? c.i : c.i * n2 + c.j;
  return c;
}
__device__ __forceinline__ int ceil_log2(int n) { return n > 1 ? 32 - __clz(n - 1) : 0; }

// One gradient's loop nest over the rows of g in the window [wlo, whi] (as values of m = m1 + m2):
//     for every own row o:   emit(o + lo_own,  sum_q  C[o,q] g[o+q] conj(other[q]))
// with (o, q) = (m1, m2) for the gradient of x and (m2, m1) for the gradient of y; `other` is the other operand's
// part in LDS (rows nq apart) and pos the start of the matching coefficient stream.
template <int CAP, class E>
__device__ __forceinline__ void gradient_pass(const RowRegs<CAP> &G, int wlo, int whi, int l_own, int l_other, int l,
                                              LdsC other, int nq, const float *bank, int pos, int lane, E &&emit) {
  CoeffStream cs;
  cs.start(bank, pos, lane);
  for (int o = -l_own; o <= l_own; o++) {
    const int qlo = max(-l_other, -l - o), qhi = min(l_other, l - o);
    if (qlo > qhi) continue;
    const int lo = max(qlo, wlo - o), hi = min(qhi, whi - o);
    const int row_pos = pos + (lo - qlo);
    pos += qhi - qlo + 1;
    if (lo > hi) continue;
    LdsC qp = other + (lo + l_other) * nq;
    int k = o + lo - wlo;  // row inside the window
    float ar = 0.f, ai = 0.f;
    for_coeffs(cs, row_pos, hi - lo + 1, lane, [&](float c) __attribute__((always_inline)) {
      float gr, gi;
      G.get(k, gr, gi);
      const v2f v = *qp;
      k++;
      qp += nq;
      const float pr = c * gr, pi = c * gi;  // (C g) conj(other)
      ar = fmaf(pr, v.x, ar);
      ar = fmaf(pi, v.y, ar);
      ai = fmaf(pi, v.x, ai);
      ai = fmaf(-pr, v.y, ai);
    });
    emit(o + l_own, ar, ai);
  }
}

// Both gradients from one pass over g; partial sums go to gradient images in LDS with float atomics.  This is the
// form that accepts everything (any mix of channel counts, operand l up to the maximum); LDS float atomics are
// slow on this hardware, so the striped kernel below is used whenever its conditions hold.
template <int CAP, bool DIAG, bool WX, bool WY>
__global__ void __launch_bounds__(bwd_max_threads<CAP>()) staged_bwd_kernel(const StagedArgs) {
  const ArgPtr a = kernel_args();
  extern __shared__ float2 staged_lds[];
  const int cpb = a->cpb, xsize = a->xsize, ysize = a->ysize;
  float2 *xs = staged_lds;
  float2 *ys = xs + cpb * xsize;
  float2 *xacc = ys + cpb * ysize;
  float2 *yacc = xacc + cpb * xsize;
  const long long cell0 = (long long)blockIdx.x * cpb;
  const long long left = a->ncells - cell0;
  const int ncell = left < cpb ? (int)left : cpb;
  if (WY) copy_image<0>(a->x, a->xrows, a->nx, xs, xsize, cell0, ncell);
  if (WX) copy_image<0>(a->y, a->yrows, a->ny, ys, ysize, cell0, ncell);
  {
    const int nacc = cpb * (xsize + ysize);
    for (int e = threadIdx.x; e < nacc; e += blockDim.x) xacc[e] = make_float2(0.f, 0.f);
  }
  __syncthreads();

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & (kWave - 1);
  const int W = blockDim.x >> 6;
  const TriplePtr triples = (TriplePtr)a->triples;
  const float *bank = a->bank;
  const int ntriples = a->ntriples, offs_add = a->offs_add;
  RowRegs<CAP> G;
  G.clear();
  int base = 0;
  for (int t = 0; t < ntriples; t++) {
    const TriplePtr tr = triples + t;
    const int log2_u = tr->log2_u;
    const int nruns = ((cpb << log2_u) + kWave - 1) >> 6;
    const int first = first_run(base, wave, W, nruns);
    if (first >= nruns) continue;
    const int l1 = tr->l1, l2 = tr->l2, l = tr->l, n1 = tr->n1, n2 = tr->n2;
    const int span = log2_u < 6 ? (1 << log2_u) : kWave;  // lanes of a run that belong to one cell
    const FastPart P = load_part(a->r + tr->ri);
    for (int run = first; run < nruns; run += W) {
      const int flat = (run << 6) + lane;
      int cl = flat >> log2_u;
      const int u = flat & ((1 << log2_u) - 1);
      const bool live = cl < ncell;
      if (!live) cl = ncell - 1;  // dead lanes read valid memory and never add
      const int n2p = DIAG ? 1 : (1 << tr->lg_n2p);
      const LaneChan lc = lane_chan<DIAG>(u, tr->lg_n2p, n1, n2);
      const int i = lc.i, j = lc.j;
      const bool writer = live && lc.valid;
      GlobalC *gp = (GlobalC *)P.ptr + (cell0 + cl) * P.sb + (tr->offs + offs_add + lc.chan);
      const int rows = 2 * l + 1;
      // g is taken through the registers in windows of CAP rows (one window unless 2l+1 > CAP); each window adds
      // the terms whose row m1+m2 falls inside it
      for (int w0 = 0; w0 < rows; w0 += CAP) {
        load_window<CAP>(G, gp, P.sm, w0, rows, lc.valid);
        const int wlo = w0 - l, whi = w0 + CAP - 1 - l;
        if (WX) {
          LdsF *xa = (LdsF *)(xacc + cl * xsize + tr->xoff + i);
          gradient_pass<CAP>(G, wlo, whi, l1, l2, l, (LdsC)ys + (cl * ysize + tr->yoff + j), n2, bank, tr->cg_back0,
                             lane, [&](int row, float ar, float ai) __attribute__((always_inline)) {
                               float2 acc[1] = {make_float2(ar, ai)};
                               if (!DIAG) group_sum(acc, n2p);
                               if (writer && (DIAG || j == 0)) {
                                 LdsF *dst = xa + 2 * row * n1;
                                 __hip_atomic_fetch_add(dst, acc[0].x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                                 __hip_atomic_fetch_add(dst + 1, acc[0].y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                               }
                             });
        }
        if (WY) {
          LdsF *ya = (LdsF *)(yacc + cl * ysize + tr->yoff + j);
          gradient_pass<CAP>(G, wlo, whi, l2, l1, l, (LdsC)xs + (cl * xsize + tr->xoff + i), n1, bank, tr->cg_back1,
                             lane, [&](int row, float ar, float ai) __attribute__((always_inline)) {
                               float2 acc[1] = {make_float2(ar, ai)};
                               if (!DIAG) stride_sum(acc, n2p, span);
                               if (writer && (DIAG || (u & (span - 1)) < n2p)) {
                                 LdsF *dst = ya + 2 * row * n2;
                                 __hip_atomic_fetch_add(dst, acc[0].x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                                 __hip_atomic_fetch_add(dst + 1, acc[0].y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                               }
                             });
        }
      }
    }
  }

  __syncthreads();
  if (a->accumulate) {
    if (WX) copy_image<2>(a->xg, a->xrows, a->nx, xacc, xsize, cell0, ncell);
    if (WY) copy_image<2>(a->yg, a->yrows, a->ny, yacc, ysize, cell0, ncell);
  } else {
    if (WX) copy_image<1>(a->xg, a->xrows, a->nx, xacc, xsize, cell0, ncell);
    if (WY) copy_image<1>(a->yg, a->yrows, a->ny, yacc, ysize, cell0, ncell);
  }
}

// ---- backward, pair-wise: contract over l first -------------------------------------------------------------------------
// All l of one (x part, y part) pair share x and y, so for a lane's channel pair
//     Q[m1,m2] = sum_l C_l[m1,m2] g_l[m1+m2]              (real coefficient times complex: 2 FMA per term)
//     xg[m1] += Q[m1,m2] conj(y[m2]),   yg[m2] += Q[m1,m2] conj(x[m1])      (once per (m1,m2), not once per term)
// which is ~5 instructions per term instead of ~13 for the two loop nests of the triple-wise kernel.  A wave takes
// a (pair, 64 slots) unit.  For each m it reads g_l[m] of every l of the pair into register rows (indexed by the
// position of l in the pair), walks the (m1, m-m1) of that m, and keeps both gradients of the pair in two more sets
// of register rows (indexed by m1 and m2); all three are addressed with wave-uniform run-time indices.  At the end
// of the unit the rows are summed over the lanes that share i (resp. j) and added to the block's gradient images in
// LDS with float atomics -- 2(l1+l2+1) row additions per unit, few enough not to matter.
// Conditions (host): at most CAP different l per pair, 2l1+1 and 2l2+1 at most CAP, power-of-two channel counts.
// Not the default: three sets of register rows leave one or two waves per SIMD and gathering g_l[m] over the
// pair's parts costs about as much as the arithmetic it saves (measured 6.5 ms against 5.9 ms for l1 = l2 = 10).
template <int CAP, bool DIAG, bool WX, bool WY>
__global__ void __launch_bounds__(256) staged_pair_bwd_kernel(const StagedArgs) {
  const ArgPtr a = kernel_args();
  extern __shared__ float2 staged_lds[];
  const int cpb = a->cpb, xsize = a->xsize, ysize = a->ysize;
  float2 *xs = staged_lds;
  float2 *ys = xs + cpb * xsize;
  float2 *xacc = ys + cpb * ysize;
  float2 *yacc = xacc + cpb * xsize;
  const long long cell0 = (long long)blockIdx.x * cpb;
  const long long left = a->ncells - cell0;
  const int ncell = left < cpb ? (int)left : cpb;
  if (WY) copy_image<0>(a->x, a->xrows, a->nx, xs, xsize, cell0, ncell);
  if (WX) copy_image<0>(a->y, a->yrows, a->ny, ys, ysize, cell0, ncell);
  {
    const int nacc = cpb * (xsize + ysize);
    for (int e = threadIdx.x; e < nacc; e += blockDim.x) xacc[e] = make_float2(0.f, 0.f);
  }
  __syncthreads();

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & (kWave - 1);
  const int W = blockDim.x >> 6;
  const TriplePtr triples = (TriplePtr)a->triples;
  const IntPtr pairs = (IntPtr)a->pairs;
  const float *bank = a->bank;
  const int npairs = a->npairs, offs_add = a->offs_add;
  RowRegs<CAP> G, AX, AY;
  G.clear();
  int base = 0;
  for (int pi = 0; pi < npairs; pi++) {
    const int t_first = pairs[3 * pi], nt = pairs[3 * pi + 1];
    const TriplePtr tr0 = triples + t_first;
    const int log2_u = tr0->log2_u;
    const int nruns = ((cpb << log2_u) + kWave - 1) >> 6;
    const int first = first_run(base, wave, W, nruns);
    if (first >= nruns) continue;
    const int l1 = tr0->l1, l2 = tr0->l2, n1 = tr0->n1, n2 = tr0->n2;
    const int ltop = (tr0 + (nt - 1))->l;  // l ascends inside a pair
    const int span = log2_u < 6 ? (1 << log2_u) : kWave;
    for (int run = first; run < nruns; run += W) {
      const int flat = (run << 6) + lane;
      int cl = flat >> log2_u;
      const int u = flat & ((1 << log2_u) - 1);
      const bool live = cl < ncell;
      if (!live) cl = ncell - 1;  // dead lanes read valid memory and never add
      const int n2p = DIAG ? 1 : (1 << tr0->lg_n2p);
      const LaneChan lc = lane_chan<DIAG>(u, tr0->lg_n2p, n1, n2);
      const int i = lc.i, j = lc.j;
      const bool writer = live && lc.valid;
      const LdsC xb = (LdsC)xs + (cl * xsize + tr0->xoff + i);
      const LdsC yb = (LdsC)ys + (cl * ysize + tr0->yoff + j);
      AX.clear();
      AY.clear();
      int pos = pairs[3 * pi + 2];
      CoeffStream cs;
      cs.start(bank, pos, lane);
      int tlo = 0;  // first l of the pair with l >= |m|; grows as |m| grows, so it is tracked from both ends
      for (int m = -ltop; m <= ltop; m++) {
        const int mabs = m < 0 ? -m : m;
        tlo = 0;
        while ((tr0 + tlo)->l < mabs) tlo++;
        // g_l[m] of every l of the pair.  Slots past the pair's last l repeat it, rows outside an l's range are
        // clamped into it (never used): the loads stay unconditional and the register rows one chain of writes.
        static_for<CAP>([&](auto tc) __attribute__((always_inline)) {
          constexpr int T = decltype(tc)::value;
          const TriplePtr tr = tr0 + min(T, nt - 1);
          const int l = tr->l;
          const FastPart P = load_part(a->r + tr->ri);
          const int row = min(max(m + l, 0), 2 * l);
          const v2f v = ((GlobalC *)P.ptr)[(cell0 + cl) * P.sb + (tr->offs + offs_add + lc.chan) + (long long)row * P.sm];
          G.template set<T>(lc.valid ? v.x : 0.f, lc.valid ? v.y : 0.f);
        });
        const int m1lo = max(-l1, m - l2), m1hi = min(l1, m + l2);
        const int len = nt - tlo;
        LdsC xp = xb + (m1lo + l1) * n1;
        LdsC yp = yb + (m - m1lo + l2) * n2;
        for (int m1 = m1lo; m1 <= m1hi; m1++, xp += n1, yp -= n2) {
          float qr = 0.f, qi = 0.f;
          int k = tlo;
          for_coeffs(cs, pos, len, lane, [&](float c) __attribute__((always_inline)) {
            float gr, gi;
            G.get(k, gr, gi);
            k++;
            qr = fmaf(c, gr, qr);
            qi = fmaf(c, gi, qi);
          });
          pos += len;
          if (WX) {
            const v2f yv = *yp;  // Q conj(y)
            AX.add(m1 + l1, fmaf(qr, yv.x, qi * yv.y), fmaf(qi, yv.x, -qr * yv.y));
          }
          if (WY) {
            const v2f xv = *xp;  // Q conj(x)
            AY.add(m - m1 + l2, fmaf(qr, xv.x, qi * xv.y), fmaf(qi, xv.x, -qr * xv.y));
          }
        }
      }
      // the pair's rows: sum over the lanes that share i (resp. j), then one lane of each group adds them to the image
      if (WX) {
        float2 out[CAP];
        static_for<CAP>([&](auto mc) __attribute__((always_inline)) { out[decltype(mc)::value] = AX.template row<decltype(mc)::value>(); });
        if (!DIAG) group_sum(out, n2p);
        if (writer && (DIAG || j == 0)) {
          LdsF *xa = (LdsF *)(xacc + cl * xsize + tr0->xoff + i);
          static_for<CAP>([&](auto mc) __attribute__((always_inline)) {
            constexpr int M = decltype(mc)::value;
            if (M < 2 * l1 + 1) {
              __hip_atomic_fetch_add(xa + 2 * M * n1, out[M].x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
              __hip_atomic_fetch_add(xa + 2 * M * n1 + 1, out[M].y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
          });
        }
      }
      if (WY) {
        float2 out[CAP];
        static_for<CAP>([&](auto mc) __attribute__((always_inline)) { out[decltype(mc)::value] = AY.template row<decltype(mc)::value>(); });
        if (!DIAG) stride_sum(out, n2p, span);
        if (writer && (DIAG || (u & (span - 1)) < n2p)) {
          LdsF *ya = (LdsF *)(yacc + cl * ysize + tr0->yoff + j);
          static_for<CAP>([&](auto mc) __attribute__((always_inline)) {
            constexpr int M = decltype(mc)::value;
            if (M < 2 * l2 + 1) {
              __hip_atomic_fetch_add(ya + 2 * M * n2, out[M].x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
              __hip_atomic_fetch_add(ya + 2 * M * n2 + 1, out[M].y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
          });
        }
      }
    }
  }

  __syncthreads();
  if (a->accumulate) {
    if (WX) copy_image<2>(a->xg, a->xrows, a->nx, xacc, xsize, cell0, ncell);
    if (WY) copy_image<2>(a->yg, a->yrows, a->ny, yacc, ysize, cell0, ncell);
  } else {
    if (WX) copy_image<1>(a->xg, a->xrows, a->nx, xacc, xsize, cell0, ncell);
    if (WY) copy_image<1>(a->yg, a->yrows, a->ny, yacc, ysize, cell0, ncell);
  }
}

// ---- backward, one gradient per launch, sums kept in registers ---------------------------------------------------------
// ROLE 0 computes the gradient of x, ROLE 1 that of y.  All triples that feed one part of that gradient form a
// stripe; a wave takes a (stripe, 64 channel slots) unit, walks the stripe's triples and keeps the part's rows in a
// second set of register rows (again indexed with a wave-uniform run-time row), so nothing is shared between waves:
// no atomics, no gradient image in LDS, a fixed summation order.  The sums over the lanes that share i (resp. j)
// are taken once per unit, on the finished rows, and the rows are stored straight to memory.  LDS holds only the
// other operand.  The price is that each launch reads g, i.e. g is read twice for the two gradients.
// Conditions (checked by the host): inside a stripe the other operand's channel count does not change, so a
// lane's (i, j) stays the same across the stripe's triples; own l at most (CAP-1)/2.
// Units are handed out through a counter in LDS, heaviest stripes (largest l) first.
constexpr int kStripeHeader = 2;  // complex elements in front of the operand image (holds the unit counter)

template <int CAP, bool DIAG, int ROLE>
__global__ void __launch_bounds__(256) staged_stripe_kernel(const StagedArgs) {
  const ArgPtr a = kernel_args();
  extern __shared__ float2 staged_lds[];
  // the unit counter sits in front of the image, in the dynamic allocation: with any static LDS the kernel could
  // no longer ask for the full 160 KB
  int &next_unit = *reinterpret_cast<int *>(staged_lds);
  const int cpb = a->cpb;
  const int osize = ROLE == 0 ? a->ysize : a->xsize;  // the other operand's image
  float2 *os = staged_lds + kStripeHeader;
  const long long cell0 = (long long)blockIdx.x * cpb;
  const long long left = a->ncells - cell0;
  const int ncell = left < cpb ? (int)left : cpb;
  if (ROLE == 0) copy_image<0>(a->y, a->yrows, a->ny, os, osize, cell0, ncell);
  else copy_image<0>(a->x, a->xrows, a->nx, os, osize, cell0, ncell);
  if (threadIdx.x == 0) next_unit = 0;
  __syncthreads();

  const int lane = threadIdx.x & (kWave - 1);
  const TriplePtr triples = (TriplePtr)a->triples;
  const float *bank = a->bank;
  const int offs_add = a->offs_add;
  const bool accumulate = a->accumulate != 0;
  const int nstripes = ROLE == 0 ? a->nx : a->ny;
  const IntPtr table = (IntPtr)a->stripes + (ROLE == 0 ? 0 : 3 * a->nx);  // (first, count, log2 slots) per stripe
  const IntPtr order = (IntPtr)a->stripes + 3 * (a->nx + a->ny) + (ROLE == 0 ? 0 : a->ntriples);
  RowRegs<CAP> G, A;
  G.clear();
  for (;;) {
    int idx = 0;
    if (lane == 0) idx = __hip_atomic_fetch_add(&next_unit, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    idx = __builtin_amdgcn_readfirstlane(idx);
    // which stripe: the last (largest l) first
    int k = nstripes - 1, log2_u = 0;
    for (; k >= 0; k--) {
      log2_u = table[3 * k + 2];
      const int units = log2_u >= 6 ? cpb : (((cpb << log2_u) + kWave - 1) >> 6);
      if (idx < units) break;
      idx -= units;
    }
    if (k < 0) break;  // every unit has been taken: the counter only grows, so every wave gets here
    const int first = table[3 * k], count = table[3 * k + 1];
    const FastPart OWN = load_part((ROLE == 0 ? a->xg : a->yg) + k);
    const int own_rows = ROLE == 0 ? a->xrows[k] : a->yrows[k];
    const int nsub = log2_u >= 6 ? (1 << (log2_u - 6)) : 1;  // runs of 64 slots inside one cell
    const int span = log2_u < 6 ? (1 << log2_u) : kWave;
    // channel count of the other operand, the same for the whole stripe (1 for a stripe without triples)
    int n_other = 1;
    if (count > 0) {
      const TriplePtr t0 = triples + order[first];
      n_other = ROLE == 0 ? t0->n2 : t0->n1;
    }
    const int n_own = OWN.n;
    const int n1 = ROLE == 0 ? n_own : n_other, n2 = ROLE == 0 ? n_other : n_own;
    const int lg_n2 = DIAG ? 0 : ceil_log2(n2);
    const int n2p = 1 << lg_n2;
    A.clear();
    for (int sub = 0; sub < nsub; sub++) {
      const int flat = log2_u >= 6 ? ((idx << log2_u) + (sub << 6) + lane) : ((idx << 6) + lane);
      int cl = flat >> log2_u;
      const int u = flat & ((1 << log2_u) - 1);
      const bool live = cl < ncell;
      if (!live) cl = ncell - 1;  // dead lanes read valid memory and never store
      const LaneChan lc = lane_chan<DIAG>(u, lg_n2, n1, n2);
      const int i = lc.i, j = lc.j;
      for (int t = 0; t < count; t++) {
        const TriplePtr tr = triples + order[first + t];
        const int l1 = tr->l1, l2 = tr->l2, l = tr->l;
        const FastPart P = load_part(a->r + tr->ri);
        GlobalC *gp = (GlobalC *)P.ptr + (cell0 + cl) * P.sb + (tr->offs + offs_add + lc.chan);
        const int rows = 2 * l + 1;
        for (int w0 = 0; w0 < rows; w0 += CAP) {
          load_window<CAP>(G, gp, P.sm, w0, rows, lc.valid);
          const int wlo = w0 - l, whi = w0 + CAP - 1 - l;
          auto add_row = [&](int row, float ar, float ai) __attribute__((always_inline)) { A.add(row, ar, ai); };
          if (ROLE == 0)
            gradient_pass<CAP>(G, wlo, whi, l1, l2, l, (LdsC)os + (cl * osize + tr->yoff + j), n2, bank, tr->cg_back0,
                               lane, add_row);
          else
            gradient_pass<CAP>(G, wlo, whi, l2, l1, l, (LdsC)os + (cl * osize + tr->xoff + i), n1, bank, tr->cg_back1,
                               lane, add_row);
        }
      }
      // the gradient of x is complete for this run's i; the gradient of y still sums over the other runs' i
      if (ROLE == 1 && !DIAG && sub + 1 < nsub) continue;
      float2 out[CAP];
      static_for<CAP>([&](auto mc) __attribute__((always_inline)) {
        constexpr int M = decltype(mc)::value;
        out[M] = A.template row<M>();
      });
      bool writer = live && lc.valid;
      int column = ROLE == 0 ? i : j;
      if (!DIAG) {
        if (ROLE == 0) {
          group_sum(out, n2p);
          writer = writer && j == 0;
        } else {
          // the sum over i ran over every run of the cell, so whether this lane writes depends on its j alone
          // (the same in every run), not on the i of the last run
          stride_sum(out, n2p, span);
          column = u & (n2p - 1);
          writer = live && column < n2 && (u & (span - 1)) < n2p;
        }
      }
      GlobalC *dst = (GlobalC *)OWN.ptr + (cell0 + cl) * OWN.sb + column;
      if (writer) {
        static_for<CAP>([&](auto mc) __attribute__((always_inline)) {
          constexpr int M = decltype(mc)::value;
          if (M < own_rows) {
            v2f o = {out[M].x, out[M].y};
            if (accumulate) o += dst[(long long)M * OWN.sm];
            dst[(long long)M * OWN.sm] = o;
          }
        });
      }
      A.clear();
    }
  }
}

constexpr int kMaxDynamicLds = 160 * 1024;

template <class K>
int launch(K kern, const StagedArgs &a, int threads, int nblocks, size_t lds, hipStream_t s, bool *attr_set) {
  if (!*attr_set) {  // benign race: setting the attribute twice is harmless
    GELIB_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      kMaxDynamicLds));
    *attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3(nblocks), dim3(threads), lds, s, a);
  GELIB_HIP_TRY(hipGetLastError());
  return GELIB_HIP_OK;
}

template <int CAP, bool DIAG, bool WX, bool WY>
int launch_bwd_variant(const StagedArgs &a, int threads, int nblocks, size_t lds, hipStream_t s) {
  static bool attr_set = false;
  if (threads > bwd_max_threads<CAP>()) return GELIB_HIP_ERR_ARG;
  return launch(staged_bwd_kernel<CAP, DIAG, WX, WY>, a, threads, nblocks, lds, s, &attr_set);
}

template <int CAP, bool DIAG>
int launch_bwd_wants(const StagedArgs &a, bool wx, bool wy, int threads, int nblocks, size_t lds, hipStream_t s) {
  if (wx && wy) return launch_bwd_variant<CAP, DIAG, true, true>(a, threads, nblocks, lds, s);
  if (wx) return launch_bwd_variant<CAP, DIAG, true, false>(a, threads, nblocks, lds, s);
  return launch_bwd_variant<CAP, DIAG, false, true>(a, threads, nblocks, lds, s);
}

template <bool DIAG>
int launch_bwd_caps(const StagedArgs &a, bool wx, bool wy, int cap, int threads, int nblocks, size_t lds,
                    hipStream_t s) {
  switch (cap) {
    case 16: return launch_bwd_wants<16, DIAG>(a, wx, wy, threads, nblocks, lds, s);
    case 32: return launch_bwd_wants<32, DIAG>(a, wx, wy, threads, nblocks, lds, s);
  }
  return GELIB_HIP_ERR_ARG;
}

template <int CAP, bool DIAG, bool WX, bool WY>
int launch_pair_variant(const StagedArgs &a, int nblocks, size_t lds, hipStream_t s) {
  static bool attr_set = false;
  return launch(staged_pair_bwd_kernel<CAP, DIAG, WX, WY>, a, 256, nblocks, lds, s, &attr_set);
}

template <int CAP, bool DIAG>
int launch_pair_wants(const StagedArgs &a, bool wx, bool wy, int nblocks, size_t lds, hipStream_t s) {
  if (wx && wy) return launch_pair_variant<CAP, DIAG, true, true>(a, nblocks, lds, s);
  if (wx) return launch_pair_variant<CAP, DIAG, true, false>(a, nblocks, lds, s);
  return launch_pair_variant<CAP, DIAG, false, true>(a, nblocks, lds, s);
}

template <int CAP, bool DIAG, int ROLE>
int launch_stripe_variant(const StagedArgs &a, int nblocks, size_t lds, hipStream_t s) {
  static bool attr_set = false;
  return launch(staged_stripe_kernel<CAP, DIAG, ROLE>, a, 256, nblocks, lds, s, &attr_set);
}

template <int CAP>
int launch_stripe_cap(const StagedArgs &a, bool diag, int role, int nblocks, size_t lds, hipStream_t s) {
  if (diag) return role == 0 ? launch_stripe_variant<CAP, true, 0>(a, nblocks, lds, s)
                             : launch_stripe_variant<CAP, true, 1>(a, nblocks, lds, s);
  return role == 0 ? launch_stripe_variant<CAP, false, 0>(a, nblocks, lds, s)
                   : launch_stripe_variant<CAP, false, 1>(a, nblocks, lds, s);
}

}  // namespace

template <bool DIAG, bool LDSC>
static int launch_fwd_tiles(const StagedArgs &a, int tile, int threads, int nblocks, size_t lds, hipStream_t s) {
  static bool attr[3] = {false, false, false};
  if (tile == 4) return launch(staged_fwd_kernel<DIAG, 4, LDSC>, a, threads, nblocks, lds, s, &attr[0]);
  if (tile == 2) return launch(staged_fwd_kernel<DIAG, 2, LDSC>, a, threads, nblocks, lds, s, &attr[1]);
  if (tile == 1) return launch(staged_fwd_kernel<DIAG, 1, LDSC>, a, threads, nblocks, lds, s, &attr[2]);
  return GELIB_HIP_ERR_ARG;
}

int launch_staged_fwd(const StagedArgs &a, bool diag, int tile, int threads, int nblocks, size_t lds_bytes,
                      hipStream_t s) {
  if (lds_bytes > (size_t)kMaxDynamicLds || threads < 64 || threads > 1024 || threads % 64) return GELIB_HIP_ERR_ARG;
  const bool ldsc = a.lds_coeffs > 0;
  if (diag) return ldsc ? launch_fwd_tiles<true, true>(a, tile, threads, nblocks, lds_bytes, s)
                        : launch_fwd_tiles<true, false>(a, tile, threads, nblocks, lds_bytes, s);
  return ldsc ? launch_fwd_tiles<false, true>(a, tile, threads, nblocks, lds_bytes, s)
              : launch_fwd_tiles<false, false>(a, tile, threads, nblocks, lds_bytes, s);
}

int launch_staged_bwd(const StagedArgs &a, bool diag, bool want_x, bool want_y, int cap, int threads, int nblocks,
                      size_t lds_bytes, hipStream_t s) {
  if (lds_bytes > (size_t)kMaxDynamicLds || (!want_x && !want_y)) return GELIB_HIP_ERR_ARG;
  if (diag) return launch_bwd_caps<true>(a, want_x, want_y, cap, threads, nblocks, lds_bytes, s);
  return launch_bwd_caps<false>(a, want_x, want_y, cap, threads, nblocks, lds_bytes, s);
}

int launch_staged_stripe(const StagedArgs &a, bool diag, int role, int cap, int nblocks, size_t lds_bytes,
                         hipStream_t s) {
  lds_bytes += kStripeHeader * sizeof(float2);
  if (lds_bytes > (size_t)kMaxDynamicLds || (role != 0 && role != 1)) return GELIB_HIP_ERR_ARG;
  if (cap == 16) return launch_stripe_cap<16>(a, diag, role, nblocks, lds_bytes, s);
  if (cap == 32) return launch_stripe_cap<32>(a, diag, role, nblocks, lds_bytes, s);
  return GELIB_HIP_ERR_ARG;
}

int launch_staged_pair_bwd(const StagedArgs &a, bool diag, bool want_x, bool want_y, int cap, int nblocks,
                           size_t lds_bytes, hipStream_t s) {
  if (lds_bytes > (size_t)kMaxDynamicLds || (!want_x && !want_y)) return GELIB_HIP_ERR_ARG;
  if (cap == 16) return diag ? launch_pair_wants<16, true>(a, want_x, want_y, nblocks, lds_bytes, s)
                             : launch_pair_wants<16, false>(a, want_x, want_y, nblocks, lds_bytes, s);
  if (cap == 32) return diag ? launch_pair_wants<32, true>(a, want_x, want_y, nblocks, lds_bytes, s)
                             : launch_pair_wants<32, false>(a, want_x, want_y, nblocks, lds_bytes, s);
  return GELIB_HIP_ERR_ARG;
}

}  // namespace gelib_hip
