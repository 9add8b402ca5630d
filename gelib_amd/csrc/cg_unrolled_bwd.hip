// Backward CG / DiagCG product for l1, l2 <= kLT: both gradients from one pass over g, all triples in one launch.
//
// Work split: every wave owns whole cells (one cell, or 64/U cells when a cell has U < 64 channel slots) and walks
// all (l1,l2) pairs for them, so no reduction ever crosses a wave and the kernel has no barrier after the
// coefficient bank is staged.  A lane owns one channel pair (i, j) of the gradient block: it reads g[m, i*n2+j]
// for every m (contiguous across the wave), forms C*g once per (m1,m2) and feeds two complex FMAs,
//     ax[m1] += (C g) conj(y[m2, j])        ay[m2] += (C g) conj(x[m1, i]),
// with all m-loops unrolled and x, y, ax, ay in registers.  ax is then summed over j with butterfly shuffles
// inside aligned groups of n2 lanes, ay over i with butterflies at lane distance n2 and up; one lane per group
// adds the result into the wave's private image of xg / yg in LDS (plain read-add-write, fixed order, no
// atomics).  After the last pair the wave writes its image to memory in contiguous rows.
#include <type_traits>
#include <utility>

#include "cg_unrolled_dev.h"

namespace gelib_hip {

namespace {

constexpr int cabs_(int a) { return a < 0 ? -a : a; }
constexpr int cmin_(int a, int b) { return a < b ? a : b; }

template <int L1, int L2, int L, bool WX, bool WY>
__device__ __forceinline__ void triple_bwd(const float2 (&xv)[2 * L1 + 1], const float2 (&yv)[2 * L2 + 1],
                                           float2 (&ax)[2 * L1 + 1], float2 (&ay)[2 * L2 + 1],
                                           const float *__restrict__ C, const float2 *__restrict__ gp, int sm) {
  float2 g[2 * L + 1];
#pragma unroll
  for (int m = 0; m <= 2 * L; m++) g[m] = gp[m * sm];
#pragma unroll
  for (int m1 = -L1; m1 <= L1; m1++) {
#pragma unroll
    for (int m2 = -L2; m2 <= L2; m2++) {
      const int m = m1 + m2;
      if (m >= -L && m <= L) {
        const float c = C[(m1 + L1) * (2 * L2 + 1) + (m2 + L2)];
        const float tr = c * g[m + L].x, ti = c * g[m + L].y;
        if (WX) {
          const float2 yc = yv[m2 + L2];
          ax[m1 + L1].x = fmaf(tr, yc.x, ax[m1 + L1].x);
          ax[m1 + L1].x = fmaf(ti, yc.y, ax[m1 + L1].x);
          ax[m1 + L1].y = fmaf(ti, yc.x, ax[m1 + L1].y);
          ax[m1 + L1].y = fmaf(-tr, yc.y, ax[m1 + L1].y);
        }
        if (WY) {
          const float2 xc = xv[m1 + L1];
          ay[m2 + L2].x = fmaf(tr, xc.x, ay[m2 + L2].x);
          ay[m2 + L2].x = fmaf(ti, xc.y, ay[m2 + L2].x);
          ay[m2 + L2].y = fmaf(ti, xc.x, ay[m2 + L2].y);
          ay[m2 + L2].y = fmaf(-tr, xc.y, ay[m2 + L2].y);
        }
      }
    }
  }
}

// The wave's view of one pair: operand parts and the gradient part of each l, picked out of the kernel arguments
// once per pair, plus the few scalars the pair code needs.
struct PairParts {
  FastPart X, Y;
  FastPart G[kMaxDl];
  long long ncells;
  int xsize, ysize, log2_u, offs_add;
};

template <int L1, int L2, bool DIAG, bool WX, bool WY>
__device__ __forceinline__ void pair_bwd(const PairParts &a, const PairRec &p, const float *Cs, float2 *xacc,
                                         float2 *yacc, long long cell_base, int lane) {
  const int N1 = p.n1, N2 = p.n2;
  const int U = DIAG ? N1 : N1 * N2;
  const int lg_n2 = DIAG ? 0 : 31 - __clz(N2);
  const int span = U < kWave ? U : kWave;           // lanes that belong to one cell
  const int sub = U < kWave ? (lane >> a.log2_u) : 0;
  const int lane_in_cell = lane & (span - 1);
  const long long cell = cell_base + sub;
  const bool live = cell < a.ncells;
  const long long cellc = live ? cell : a.ncells - 1;
  const FastPart X = a.X;
  const FastPart Y = a.Y;
  float2 *xa = xacc + sub * a.xsize + p.xoff;
  float2 *ya = yacc + sub * a.ysize + p.yoff;
  const int nchunk = U < kWave ? 1 : U >> 6;
  for (int ch = 0; ch < nchunk; ch++) {
    const int u = (ch << 6) + lane_in_cell;
    const int i = DIAG ? u : (u >> lg_n2);
    const int j = DIAG ? u : (u & (N2 - 1));
    float2 xv[2 * L1 + 1], yv[2 * L2 + 1], ax[2 * L1 + 1], ay[2 * L2 + 1];
    if (WY) {
      const float2 *xp = X.ptr + cellc * X.sb + i;
#pragma unroll
      for (int m1 = 0; m1 <= 2 * L1; m1++) xv[m1] = xp[m1 * X.sm];
    }
    if (WX) {
      const float2 *yp = Y.ptr + cellc * Y.sb + j;
#pragma unroll
      for (int m2 = 0; m2 <= 2 * L2; m2++) yv[m2] = yp[m2 * Y.sm];
    }
#pragma unroll
    for (int m1 = 0; m1 <= 2 * L1; m1++) ax[m1] = make_float2(0.f, 0.f);
#pragma unroll
    for (int m2 = 0; m2 <= 2 * L2; m2++) ay[m2] = make_float2(0.f, 0.f);

    constexpr int LMIN = cabs_(L1 - L2);
    constexpr int NL = 2 * cmin_(L1, L2) + 1;
    static_for<NL>([&](auto dl_c) __attribute__((always_inline)) {
      constexpr int dl = decltype(dl_c)::value;
      constexpr int L = LMIN + dl;
      if (p.ri[dl] >= 0) {
        const FastPart G = a.G[dl];
        const float2 *gp = G.ptr + cellc * G.sb + (p.offs[dl] + a.offs_add + u);
        triple_bwd<L1, L2, L, WX, WY>(xv, yv, ax, ay, Cs + p.cg[dl], gp, G.sm);
      }
    });

    if (WX) {
#pragma unroll
      for (int m1 = 0; m1 <= 2 * L1; m1++) {
        float2 v = ax[m1];
        if (!DIAG)
          for (int s = 1; s < N2; s <<= 1) {
            v.x += __shfl_xor(v.x, s);
            v.y += __shfl_xor(v.y, s);
          }
        if (live && (DIAG || j == 0)) {
          float2 *d = xa + m1 * N1 + i;
          float2 o = *d;
          o.x += v.x;
          o.y += v.y;
          *d = o;
        }
      }
    }
    if (WY) {
#pragma unroll
      for (int m2 = 0; m2 <= 2 * L2; m2++) {
        float2 v = ay[m2];
        if (!DIAG)
          for (int s = N2; s < span; s <<= 1) {
            v.x += __shfl_xor(v.x, s);
            v.y += __shfl_xor(v.y, s);
          }
        if (live && (DIAG || lane_in_cell < N2)) {
          float2 *d = ya + m2 * N2 + j;
          float2 o = *d;
          o.x += v.x;
          o.y += v.y;
          *d = o;
        }
      }
    }
  }
}

__device__ __forceinline__ void write_image(const FastPart (&parts)[kFastIn], const int (&rows)[kFastIn], int nparts,
                                            const float2 *img, long long cell, int lane, bool accumulate) {
  int off = 0;
  static_for<kFastIn>([&](auto kc) __attribute__((always_inline)) {
    constexpr int k = decltype(kc)::value;
    if (k < nparts) {
      const FastPart P = parts[k];
      const int total = rows[k] * P.n;
      float2 *base = P.ptr + cell * P.sb;
      for (int e = lane; e < total; e += kWave) {
        const int m = e / P.n;
        const int c = e - m * P.n;
        float2 v = img[off + e];
        float2 *d = base + m * P.sm + c;
        if (accumulate) {
          const float2 o = *d;
          v.x += o.x;
          v.y += o.y;
        }
        *d = v;
      }
      off += total;
    }
  });
}

template <bool DIAG, bool WX, bool WY>
__global__ void __launch_bounds__(kBlock) unrolled_bwd_kernel(const BwdArgs a) {
  extern __shared__ float lds[];
  float *Cs = lds;
  for (int i = threadIdx.x; i < a.bank_len; i += kBlock) Cs[i] = a.bank[i];
  __syncthreads();

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & (kWave - 1);
  const int cpw = a.cells_per_wave;
  const int img = a.xsize + a.ysize;
  float2 *acc = reinterpret_cast<float2 *>(lds + ((a.bank_len + 1) & ~1));
  float2 *xacc = acc + wave * cpw * img;
  float2 *yacc = xacc + cpw * a.xsize;
  const long long cell_base = ((long long)blockIdx.x * (kBlock / kWave) + wave) * cpw;
  if (cell_base >= a.ncells) return;  // no barrier follows: a whole wave may leave
  for (int i = lane; i < cpw * img; i += kWave) xacc[i] = make_float2(0.f, 0.f);

  PairParts pp;
  pp.ncells = a.ncells;
  pp.xsize = a.xsize;
  pp.ysize = a.ysize;
  pp.log2_u = a.log2_u;
  pp.offs_add = a.offs_add;
  for (int pidx = 0; pidx < a.npairs; pidx++) {
    const PairRec &p = a.pairs[pidx];
    const float *C = Cs + p.cg_base;
    pp.X = pick_part(a.x, p.xi);
    pp.Y = pick_part(a.y, p.yi);
    static_for<kMaxDl>([&](auto d) __attribute__((always_inline)) { pp.G[d.value] = pick_part(a.g, p.ri[d.value]); });
    switch (p.l1 * (kLT + 1) + p.l2) {
#define GELIB_CASE(A, B) \
  case A * (kLT + 1) + B: pair_bwd<A, B, DIAG, WX, WY>(pp, p, C, xacc, yacc, cell_base, lane); break;
#define GELIB_ROW(A) GELIB_CASE(A, 0) GELIB_CASE(A, 1) GELIB_CASE(A, 2) GELIB_CASE(A, 3) GELIB_CASE(A, 4)
      GELIB_ROW(0) GELIB_ROW(1) GELIB_ROW(2) GELIB_ROW(3) GELIB_ROW(4)
#undef GELIB_ROW
#undef GELIB_CASE
      default: break;
    }
  }

  for (int sub = 0; sub < cpw; sub++) {
    const long long cell = cell_base + sub;
    if (cell >= a.ncells) break;
    if (WX) write_image(a.xg, a.xrows, a.nx, xacc + sub * a.xsize, cell, lane, a.accumulate != 0);
    if (WY) write_image(a.yg, a.yrows, a.ny, yacc + sub * a.ysize, cell, lane, a.accumulate != 0);
  }
}

template <bool DIAG, bool WX, bool WY>
int launch_variant(const BwdArgs &a, int nblocks, size_t lds, hipStream_t s) {
  auto kern = unrolled_bwd_kernel<DIAG, WX, WY>;
  static bool attr_set = false;
  if (!attr_set) {
    GELIB_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      160 * 1024));
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3(nblocks), dim3(kBlock), lds, s, a);
  GELIB_HIP_TRY(hipGetLastError());
  return GELIB_HIP_OK;
}

}  // namespace

int launch_unrolled_bwd(const BwdArgs &a, bool diag, int nblocks, size_t lds_bytes, hipStream_t s) {
  static_assert(kLT == 4, "the case table above lists l1, l2 = 0..4");
  if (nblocks <= 0) return GELIB_HIP_OK;
  const bool wx = a.want_x != 0, wy = a.want_y != 0;
  if (diag) {
    if (wx && wy) return launch_variant<true, true, true>(a, nblocks, lds_bytes, s);
    if (wx) return launch_variant<true, true, false>(a, nblocks, lds_bytes, s);
    return launch_variant<true, false, true>(a, nblocks, lds_bytes, s);
  }
  if (wx && wy) return launch_variant<false, true, true>(a, nblocks, lds_bytes, s);
  if (wx) return launch_variant<false, true, false>(a, nblocks, lds_bytes, s);
  return launch_variant<false, false, true>(a, nblocks, lds_bytes, s);
}

}  // namespace gelib_hip
