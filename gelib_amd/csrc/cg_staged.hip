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

// ---- forward ------------------------------------------------------------------------------------------------------
template <bool DIAG>
__global__ void __launch_bounds__(256) staged_fwd_kernel(const StagedArgs) {
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
  __syncthreads();

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & (kWave - 1);
  const int W = blockDim.x >> 6;
  const TriplePtr triples = (TriplePtr)a->triples;
  const CoeffPtr bank = (CoeffPtr)a->bank;
  const int ntriples = a->ntriples, offs_add = a->offs_add;
  const bool accumulate = a->accumulate != 0;
  int base = 0;
  for (int t = 0; t < ntriples; t++) {
    const TriplePtr tr = triples + t;
    const int U = tr->u;
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
      const int u = fc - cl * U;
      const int i = DIAG ? u : u / n2;
      const int j = DIAG ? u : u - i * n2;
      const float2 *xb = xs + cl * xsize + tr->xoff + i;
      const float2 *yb = ys + cl * ysize + tr->yoff + j;
      GlobalC *rp = (GlobalC *)R.ptr + (cell0 + cl) * R.sb + (tr->offs + offs_add + u);
      CoeffPtr cp = bank + tr->cg_fwd;
      for (int m = -l; m <= l; m++) {
        const int m1lo = max(-l1, m - l2), m1hi = min(l1, m + l2);
        const float2 *xp = xb + (m1lo + l1) * n1;
        const float2 *yp = yb + (m - m1lo + l2) * n2;
        float ar = 0.f, ai = 0.f;
        for (int m1 = m1lo; m1 <= m1hi; m1++) {
          const float c = *cp++;
          const float2 xv = *xp, yv = *yp;
          xp += n1;
          yp -= n2;
          const float pr = c * xv.x, pi = c * xv.y;  // (C x) y, the reference's order
          ar = fmaf(pr, yv.x, ar);
          ar = fmaf(-pi, yv.y, ar);
          ai = fmaf(pr, yv.y, ai);
          ai = fmaf(pi, yv.x, ai);
        }
        if (live) {
          GlobalC *dst = rp + (long long)(m + l) * R.sm;
          v2f o = {ar, ai};
          if (accumulate) o += *dst;
          *dst = o;
        }
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
};

template <int CAP>
constexpr int bwd_max_threads() {
  return CAP == 16 ? 1024 : 512;
}

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
  const CoeffPtr bank = (CoeffPtr)a->bank;
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
      const int lg_n2 = DIAG ? 0 : 31 - __clz(n2);
      const int i = DIAG ? u : (u >> lg_n2);
      const int j = DIAG ? u : (u & (n2 - 1));
      GlobalC *gp = (GlobalC *)P.ptr + (cell0 + cl) * P.sb + (tr->offs + offs_add + u);
      const int rows = 2 * l + 1;
      // g is taken through the registers in windows of CAP rows (one window unless 2l+1 > CAP); each window adds
      // the terms whose row m1+m2 falls inside it
      for (int w0 = 0; w0 < rows; w0 += CAP) {
        static_for<CAP>([&](auto mc) __attribute__((always_inline)) {
          constexpr int M = decltype(mc)::value;
          // rows past the end repeat the last one (never used): the loads stay unconditional, which keeps the
          // register rows one straight chain of writes instead of a merge of alternatives at every row
          const int row = min(w0 + M, rows - 1);
          const v2f v = gp[(long long)row * P.sm];
          G.template set<M>(v.x, v.y);
        });
        const int wlo = w0 - l, whi = w0 + CAP - 1 - l;  // the window as a range of m = m1 + m2

        if (WX) {
          const float2 *yb = ys + cl * ysize + tr->yoff + j;
          LdsF *xa = (LdsF *)(xacc + cl * xsize + tr->xoff + i);
          CoeffPtr cp = bank + tr->cg_back0;
          for (int m1 = -l1; m1 <= l1; m1++) {
            const int m2lo = max(-l2, -l - m1), m2hi = min(l2, l - m1);
            if (m2lo > m2hi) continue;
            const int lo = max(m2lo, wlo - m1), hi = min(m2hi, whi - m1);
            CoeffPtr cq = cp + (lo - m2lo);
            cp += m2hi - m2lo + 1;
            if (lo > hi) continue;
            const float2 *yp = yb + (lo + l2) * n2;
            int k = m1 + lo - wlo;  // row inside the window
            float2 acc[1] = {make_float2(0.f, 0.f)};
            for (int m2 = lo; m2 <= hi; m2++, k++, yp += n2) {
              const float c = *cq++;
              float gr, gi;
              G.get(k, gr, gi);
              const float2 yv = *yp;
              const float pr = c * gr, pi = c * gi;  // (C g) conj(y)
              acc[0].x = fmaf(pr, yv.x, acc[0].x);
              acc[0].x = fmaf(pi, yv.y, acc[0].x);
              acc[0].y = fmaf(pi, yv.x, acc[0].y);
              acc[0].y = fmaf(-pr, yv.y, acc[0].y);
            }
            if (!DIAG) group_sum(acc, n2);
            if (live && (DIAG || j == 0)) {
              LdsF *dst = xa + 2 * (m1 + l1) * n1;
              __hip_atomic_fetch_add(dst, acc[0].x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
              __hip_atomic_fetch_add(dst + 1, acc[0].y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
          }
        }
        if (WY) {
          const float2 *xb = xs + cl * xsize + tr->xoff + i;
          LdsF *ya = (LdsF *)(yacc + cl * ysize + tr->yoff + j);
          CoeffPtr cp = bank + tr->cg_back1;
          for (int m2 = -l2; m2 <= l2; m2++) {
            const int m1lo = max(-l1, -l - m2), m1hi = min(l1, l - m2);
            if (m1lo > m1hi) continue;
            const int lo = max(m1lo, wlo - m2), hi = min(m1hi, whi - m2);
            CoeffPtr cq = cp + (lo - m1lo);
            cp += m1hi - m1lo + 1;
            if (lo > hi) continue;
            const float2 *xp = xb + (lo + l1) * n1;
            int k = lo + m2 - wlo;
            float2 acc[1] = {make_float2(0.f, 0.f)};
            for (int m1 = lo; m1 <= hi; m1++, k++, xp += n1) {
              const float c = *cq++;
              float gr, gi;
              G.get(k, gr, gi);
              const float2 xv = *xp;
              const float pr = c * gr, pi = c * gi;  // (C g) conj(x)
              acc[0].x = fmaf(pr, xv.x, acc[0].x);
              acc[0].x = fmaf(pi, xv.y, acc[0].x);
              acc[0].y = fmaf(pi, xv.x, acc[0].y);
              acc[0].y = fmaf(-pr, xv.y, acc[0].y);
            }
            if (!DIAG) stride_sum(acc, n2, span);
            if (live && (DIAG || (u & (span - 1)) < n2)) {
              LdsF *dst = ya + 2 * (m2 + l2) * n2;
              __hip_atomic_fetch_add(dst, acc[0].x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
              __hip_atomic_fetch_add(dst + 1, acc[0].y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
          }
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

}  // namespace

int launch_staged_fwd(const StagedArgs &a, bool diag, int nblocks, size_t lds_bytes, hipStream_t s) {
  static bool attr_cg = false, attr_diag = false;
  if (lds_bytes > (size_t)kMaxDynamicLds) return GELIB_HIP_ERR_ARG;
  if (diag) return launch(staged_fwd_kernel<true>, a, 256, nblocks, lds_bytes, s, &attr_diag);
  return launch(staged_fwd_kernel<false>, a, 256, nblocks, lds_bytes, s, &attr_cg);
}

int launch_staged_bwd(const StagedArgs &a, bool diag, bool want_x, bool want_y, int cap, int threads, int nblocks,
                      size_t lds_bytes, hipStream_t s) {
  if (lds_bytes > (size_t)kMaxDynamicLds || (!want_x && !want_y)) return GELIB_HIP_ERR_ARG;
  if (diag) return launch_bwd_caps<true>(a, want_x, want_y, cap, threads, nblocks, lds_bytes, s);
  return launch_bwd_caps<false>(a, want_x, want_y, cap, threads, nblocks, lds_bytes, s);
}

}  // namespace gelib_hip
