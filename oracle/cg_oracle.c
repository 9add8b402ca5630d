/*
 * CPU oracle for the SO(3) Clebsch-Gordan product path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the algorithm of the reference's CPU path so that the HIP
 * kernels can be checked against it and so that a CPU baseline can be timed beside them.
 * Nothing in the shipped library links against, loads or calls this file; only the test-suite,
 * the smoke check and the cpu_baseline leg of the benchmark do.
 *
 * What each function follows (paths relative to the reference tree):
 *   ora_cg_coeff          SO3/SO3CGbank.hpp:72-95   (slowCG: Racah sum with lgamma, double)
 *   ora_cg_matrix         SO3/SO3CGbank.hpp:58-64   (CGmatrix: row-major (2l1+1)x(2l2+1) float)
 *   part kernels          SO3/SO3part.hpp:205-257   (CGproduct fwd / back0 / back1 loop nests)
 *                         SO3/SO3part.hpp:276-322   (DiagCGproduct fwd / back0 / back1)
 *   batch loop            core/Gpart.hpp:325-360    (for_each_cell_multi: one 2-D cell per batch entry,
 *                                                    stride 0 for a broadcast operand, core/Gpart.hpp:168-185)
 *   vec-level loops       core/Gvec.hpp:311-345, core/Gvec.hpp:358-389 (triple enumeration, running offsets)
 *   type arithmetic       core/Gtype.hpp:115-138, SO3/SO3group.hpp:43-47
 *   ora_spharm            SO3/SO3part.hpp:340-403   (add_spharm: Legendre table in float, phase recurrence in
 *                                                    complex<float>; pinned by scipy's spherical harmonics -- the
 *                                                    reference's own check, python/tests/test_spharm.py -- and the
 *                                                    printed example python/docs/source/abandoned/SO3part.rst:170-176)
 *
 * How the oracle is pinned (see tests/test_oracle_*.py): coefficients against exact sympy values,
 * the printed table in python/docs/source/SO3CG.rst:51-53, orthogonality and symmetry identities;
 * kernels against brute-force loops with sympy coefficients, a complex128 einsum, closed-form
 * special cases, Wigner-D equivariance and the adjoint identities; offsets against the type
 * known-answers in python/docs/source/abandoned/SO3type.rst:28-41.
 *
 * The float32 variants keep the reference's evaluation order: loops n1 -> n2 -> m1 -> m2, each
 * term formed as (C*x)*y in complex<float> and added straight into float32 memory.  The float64
 * variants are the same loops in double with the float-rounded coefficient table, and serve as
 * the "exact" answer when measuring float32 error.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORA_MAXL 64

/* A part tensor seen as (B, M=2l+1, N) complex numbers; strides counted in complex elements. */
typedef struct {
  void *ptr;
  int64_t B, M, N;
  int64_t sb, sm, sc;
} ora_part;

enum { ORA_CG_FWD = 0, ORA_CG_BACK0 = 1, ORA_CG_BACK1 = 2, ORA_DIAG_FWD = 3, ORA_DIAG_BACK0 = 4, ORA_DIAG_BACK1 = 5 };

static double logfact(double n) { return lgamma(n + 1.0); }

static double plusminus(int k) { return (k % 2 == 1) ? -1.0 : 1.0; }

/* <l1 m1; l2 m2 | l m1+m2> exactly as the reference evaluates it (SO3/SO3CGbank.hpp:72-95). */
double ora_cg_coeff(int l1, int l2, int l, int m1, int m2) {
  int m = m1 + m2;
  int m3 = -m;
  int t1 = l2 - m1 - l;
  int t2 = l1 + m2 - l;
  int t3 = l1 + l2 - l;
  int t4 = l1 - m1;
  int t5 = l2 + m2;
  int tmin = 0;
  if (t1 > tmin) tmin = t1;
  if (t2 > tmin) tmin = t2;
  int tmax = t3;
  if (t4 < tmax) tmax = t4;
  if (t5 < tmax) tmax = t5;

  double logA = (logfact(l1 + l2 - l) + logfact(l1 - l2 + l) + logfact(-l1 + l2 + l) - logfact(l1 + l2 + l + 1)) / 2;
  logA += (logfact(l1 + m1) + logfact(l1 - m1) + logfact(l2 + m2) + logfact(l2 - m2) + logfact(l + m3) + logfact(l - m3)) / 2;

  double wigner = 0;
  for (int t = tmin; t <= tmax; t++) {
    double logB = logfact(t) + logfact(t - t1) + logfact(t - t2) + logfact(t3 - t) + logfact(t4 - t) + logfact(t5 - t);
    wigner += plusminus(t) * exp(logA - logB);
  }
  return plusminus(l1 - l2 - m3) * plusminus(l1 - l2 + m) * sqrt((double)(2 * l + 1)) * wigner;
}

/*
 * Error-analysis aid, not part of the reference's algorithm: while the switch is on, ora_cg_matrix returns |C|.
 * Run on the moduli of the operands, the float64 loop nests then give, for every element of a result, the sum of
 * the moduli of its terms, sum |C| |a| |b|: the scale that the rounding error of a float32 evaluation of that
 * element follows, whatever the order of its additions.  Process-wide; callers switch it off again.
 */
static int abs_coeffs = 0;
void ora_set_abs_coeffs(int on) { abs_coeffs = on; }

/* Row-major (2l1+1) x (2l2+1) float table; entries with |m1+m2|>l are zero (never read by the kernels). */
int ora_cg_matrix(int l1, int l2, int l, float *out) {
  if (l1 < 0 || l2 < 0 || l < abs(l1 - l2) || l > l1 + l2) return 1;
  int L2 = 2 * l2 + 1;
  memset(out, 0, sizeof(float) * (size_t)(2 * l1 + 1) * L2);
  for (int m1 = -l1; m1 <= l1; m1++) {
    int lo = (-l2 > -l - m1) ? -l2 : -l - m1;
    int hi = (l2 < l - m1) ? l2 : l - m1;
    for (int m2 = lo; m2 <= hi; m2++) {
      float c = (float)ora_cg_coeff(l1, l2, l, m1, m2);
      out[(m1 + l1) * L2 + (m2 + l2)] = abs_coeffs ? fabsf(c) : c;
    }
  }
  return 0;
}

/* ---- one 2-D cell, both precisions -------------------------------------------------------------------------- */

#define DEFINE_CELL_KERNELS(T, SUF)                                                                                 \
  static void cell_cg_fwd_##SUF(T *r, int64_t rsm, int64_t rsc, const T *x, int64_t xsm, int64_t xsc, const T *y,  \
                                int64_t ysm, int64_t ysc, const float *C, int l1, int l2, int l, int N1, int N2,    \
                                int offs) {                                                                         \
    const int L2 = 2 * l2 + 1;                                                                                      \
    for (int n1 = 0; n1 < N1; n1++) {                                                                               \
      for (int n2 = 0; n2 < N2; n2++) {                                                                             \
        for (int m1 = -l1; m1 <= l1; m1++) {                                                                        \
          int lo = (-l2 > -l - m1) ? -l2 : -l - m1;                                                                 \
          int hi = (l2 < l - m1) ? l2 : l - m1;                                                                     \
          for (int m2 = lo; m2 <= hi; m2++) {                                                                       \
            T c = (T)C[(m1 + l1) * L2 + (m2 + l2)];                                                                 \
            const T *xp = x + 2 * ((m1 + l1) * xsm + n1 * xsc);                                                     \
            const T *yp = y + 2 * ((m2 + l2) * ysm + n2 * ysc);                                                     \
            T ar = c * xp[0], ai = c * xp[1];                                                                       \
            T tr = ar * yp[0] - ai * yp[1];                                                                         \
            T ti = ar * yp[1] + ai * yp[0];                                                                         \
            T *rp = r + 2 * ((m1 + m2 + l) * rsm + (offs + n2) * rsc);                                              \
            rp[0] += tr;                                                                                            \
            rp[1] += ti;                                                                                            \
          }                                                                                                         \
        }                                                                                                           \
      }                                                                                                             \
      offs += N2;                                                                                                   \
    }                                                                                                               \
  }                                                                                                                 \
  static void cell_cg_back0_##SUF(const T *r, int64_t rsm, int64_t rsc, T *x, int64_t xsm, int64_t xsc,            \
                                  const T *y, int64_t ysm, int64_t ysc, const float *C, int l1, int l2, int l,     \
                                  int N1, int N2, int offs) {                                                       \
    const int L2 = 2 * l2 + 1;                                                                                      \
    for (int n1 = 0; n1 < N1; n1++) {                                                                               \
      for (int n2 = 0; n2 < N2; n2++) {                                                                             \
        for (int m1 = -l1; m1 <= l1; m1++) {                                                                        \
          int lo = (-l2 > -l - m1) ? -l2 : -l - m1;                                                                 \
          int hi = (l2 < l - m1) ? l2 : l - m1;                                                                     \
          for (int m2 = lo; m2 <= hi; m2++) {                                                                       \
            T c = (T)C[(m1 + l1) * L2 + (m2 + l2)];                                                                 \
            const T *rp = r + 2 * ((m1 + m2 + l) * rsm + (offs + n2) * rsc);                                        \
            const T *yp = y + 2 * ((m2 + l2) * ysm + n2 * ysc);                                                     \
            T ar = c * rp[0], ai = c * rp[1];                                                                       \
            T br = yp[0], bi = -yp[1];                                                                              \
            T *xp = x + 2 * ((m1 + l1) * xsm + n1 * xsc);                                                           \
            xp[0] += ar * br - ai * bi;                                                                             \
            xp[1] += ar * bi + ai * br;                                                                             \
          }                                                                                                         \
        }                                                                                                           \
      }                                                                                                             \
      offs += N2;                                                                                                   \
    }                                                                                                               \
  }                                                                                                                 \
  static void cell_cg_back1_##SUF(const T *r, int64_t rsm, int64_t rsc, const T *x, int64_t xsm, int64_t xsc,      \
                                  T *y, int64_t ysm, int64_t ysc, const float *C, int l1, int l2, int l, int N1,   \
                                  int N2, int offs) {                                                               \
    const int L2 = 2 * l2 + 1;                                                                                      \
    for (int n1 = 0; n1 < N1; n1++) {                                                                               \
      for (int n2 = 0; n2 < N2; n2++) {                                                                             \
        for (int m1 = -l1; m1 <= l1; m1++) {                                                                        \
          int lo = (-l2 > -l - m1) ? -l2 : -l - m1;                                                                 \
          int hi = (l2 < l - m1) ? l2 : l - m1;                                                                     \
          for (int m2 = lo; m2 <= hi; m2++) {                                                                       \
            T c = (T)C[(m1 + l1) * L2 + (m2 + l2)];                                                                 \
            const T *rp = r + 2 * ((m1 + m2 + l) * rsm + (offs + n2) * rsc);                                        \
            const T *xp = x + 2 * ((m1 + l1) * xsm + n1 * xsc);                                                     \
            T ar = c * rp[0], ai = c * rp[1];                                                                       \
            T br = xp[0], bi = -xp[1];                                                                              \
            T *yp = y + 2 * ((m2 + l2) * ysm + n2 * ysc);                                                           \
            yp[0] += ar * br - ai * bi;                                                                             \
            yp[1] += ar * bi + ai * br;                                                                             \
          }                                                                                                         \
        }                                                                                                           \
      }                                                                                                             \
      offs += N2;                                                                                                   \
    }                                                                                                               \
  }                                                                                                                 \
  static void cell_diag_fwd_##SUF(T *r, int64_t rsm, int64_t rsc, const T *x, int64_t xsm, int64_t xsc,            \
                                  const T *y, int64_t ysm, int64_t ysc, const float *C, int l1, int l2, int l,     \
                                  int N1, int N2, int offs) {                                                       \
    (void)N2;                                                                                                       \
    const int L2 = 2 * l2 + 1;                                                                                      \
    for (int n = 0; n < N1; n++) {                                                                                  \
      for (int m1 = -l1; m1 <= l1; m1++) {                                                                          \
        int lo = (-l2 > -l - m1) ? -l2 : -l - m1;                                                                   \
        int hi = (l2 < l - m1) ? l2 : l - m1;                                                                       \
        for (int m2 = lo; m2 <= hi; m2++) {                                                                         \
          T c = (T)C[(m1 + l1) * L2 + (m2 + l2)];                                                                   \
          const T *xp = x + 2 * ((m1 + l1) * xsm + n * xsc);                                                        \
          const T *yp = y + 2 * ((m2 + l2) * ysm + n * ysc);                                                        \
          T ar = c * xp[0], ai = c * xp[1];                                                                         \
          T *rp = r + 2 * ((m1 + m2 + l) * rsm + (offs + n) * rsc);                                                 \
          rp[0] += ar * yp[0] - ai * yp[1];                                                                         \
          rp[1] += ar * yp[1] + ai * yp[0];                                                                         \
        }                                                                                                           \
      }                                                                                                             \
    }                                                                                                               \
  }                                                                                                                 \
  static void cell_diag_back0_##SUF(const T *r, int64_t rsm, int64_t rsc, T *x, int64_t xsm, int64_t xsc,          \
                                    const T *y, int64_t ysm, int64_t ysc, const float *C, int l1, int l2, int l,   \
                                    int N1, int N2, int offs) {                                                     \
    (void)N2;                                                                                                       \
    const int L2 = 2 * l2 + 1;                                                                                      \
    for (int n = 0; n < N1; n++) {                                                                                  \
      for (int m1 = -l1; m1 <= l1; m1++) {                                                                          \
        int lo = (-l2 > -l - m1) ? -l2 : -l - m1;                                                                   \
        int hi = (l2 < l - m1) ? l2 : l - m1;                                                                       \
        for (int m2 = lo; m2 <= hi; m2++) {                                                                         \
          T c = (T)C[(m1 + l1) * L2 + (m2 + l2)];                                                                   \
          const T *rp = r + 2 * ((m1 + m2 + l) * rsm + (offs + n) * rsc);                                           \
          const T *yp = y + 2 * ((m2 + l2) * ysm + n * ysc);                                                        \
          T ar = c * rp[0], ai = c * rp[1];                                                                         \
          T br = yp[0], bi = -yp[1];                                                                                \
          T *xp = x + 2 * ((m1 + l1) * xsm + n * xsc);                                                              \
          xp[0] += ar * br - ai * bi;                                                                               \
          xp[1] += ar * bi + ai * br;                                                                               \
        }                                                                                                           \
      }                                                                                                             \
    }                                                                                                               \
  }                                                                                                                 \
  static void cell_diag_back1_##SUF(const T *r, int64_t rsm, int64_t rsc, const T *x, int64_t xsm, int64_t xsc,    \
                                    T *y, int64_t ysm, int64_t ysc, const float *C, int l1, int l2, int l, int N1, \
                                    int N2, int offs) {                                                             \
    (void)N2;                                                                                                       \
    const int L2 = 2 * l2 + 1;                                                                                      \
    for (int n = 0; n < N1; n++) {                                                                                  \
      for (int m1 = -l1; m1 <= l1; m1++) {                                                                          \
        int lo = (-l2 > -l - m1) ? -l2 : -l - m1;                                                                   \
        int hi = (l2 < l - m1) ? l2 : l - m1;                                                                       \
        for (int m2 = lo; m2 <= hi; m2++) {                                                                         \
          T c = (T)C[(m1 + l1) * L2 + (m2 + l2)];                                                                   \
          const T *rp = r + 2 * ((m1 + m2 + l) * rsm + (offs + n) * rsc);                                           \
          const T *xp = x + 2 * ((m1 + l1) * xsm + n * xsc);                                                        \
          T ar = c * rp[0], ai = c * rp[1];                                                                         \
          T br = xp[0], bi = -xp[1];                                                                                \
          T *yp = y + 2 * ((m2 + l2) * ysm + n * ysc);                                                              \
          yp[0] += ar * br - ai * bi;                                                                               \
          yp[1] += ar * bi + ai * br;                                                                               \
        }                                                                                                           \
      }                                                                                                             \
    }                                                                                                               \
  }                                                                                                                 \
  static int part_op_##SUF(int op, const ora_part *r, const ora_part *x, const ora_part *y, int offs,              \
                           int nthreads) {                                                                          \
    if (!(r->M & 1) || !(x->M & 1) || !(y->M & 1)) return 2;                                                        \
    int l = (int)(r->M - 1) / 2, l1 = (int)(x->M - 1) / 2, l2 = (int)(y->M - 1) / 2;                                \
    if (l < abs(l1 - l2) || l > l1 + l2 || l1 > ORA_MAXL || l2 > ORA_MAXL) return 3;                                \
    int N1 = (int)x->N, N2 = (int)y->N;                                                                             \
    int diag = (op >= ORA_DIAG_FWD);                                                                                \
    if (diag && N1 != N2) return 4;                                                                                 \
    int64_t nout = diag ? N1 : (int64_t)N1 * N2;                                                                    \
    if (offs < 0 || offs + nout > r->N) return 5;                                                                   \
    int64_t B = r->B;                                                                                               \
    if (x->B > B) B = x->B;                                                                                         \
    if (y->B > B) B = y->B;                                                                                         \
    if ((r->B != 1 && r->B != B) || (x->B != 1 && x->B != B) || (y->B != 1 && y->B != B)) return 6;                 \
    int64_t rsb = (r->B == B) ? r->sb : 0, xsb = (x->B == B) ? x->sb : 0, ysb = (y->B == B) ? y->sb : 0;            \
    float *C = (float *)malloc(sizeof(float) * (size_t)(2 * l1 + 1) * (2 * l2 + 1));                                \
    ora_cg_matrix(l1, l2, l, C);                                                                                    \
    /* a broadcast destination is summed over the batch: keep that serial */                                       \
    int dest_bcast = (op == ORA_CG_FWD || op == ORA_DIAG_FWD) ? (rsb == 0 && B > 1)                                 \
                     : (op == ORA_CG_BACK0 || op == ORA_DIAG_BACK0) ? (xsb == 0 && B > 1)                           \
                                                                    : (ysb == 0 && B > 1);                          \
    if (dest_bcast || nthreads < 1) nthreads = 1;                                                                   \
    (void)nthreads;                                                                                                 \
    _Pragma("omp parallel for num_threads(nthreads) schedule(static) if (nthreads > 1)")                            \
    for (int64_t b = 0; b < B; b++) {                                                                               \
      T *rp = (T *)r->ptr + 2 * b * rsb;                                                                            \
      T *xp = (T *)x->ptr + 2 * b * xsb;                                                                            \
      T *yp = (T *)y->ptr + 2 * b * ysb;                                                                            \
      switch (op) {                                                                                                 \
        case ORA_CG_FWD: cell_cg_fwd_##SUF(rp, r->sm, r->sc, xp, x->sm, x->sc, yp, y->sm, y->sc, C, l1, l2, l, N1, N2, offs); break;     \
        case ORA_CG_BACK0: cell_cg_back0_##SUF(rp, r->sm, r->sc, xp, x->sm, x->sc, yp, y->sm, y->sc, C, l1, l2, l, N1, N2, offs); break; \
        case ORA_CG_BACK1: cell_cg_back1_##SUF(rp, r->sm, r->sc, xp, x->sm, x->sc, yp, y->sm, y->sc, C, l1, l2, l, N1, N2, offs); break; \
        case ORA_DIAG_FWD: cell_diag_fwd_##SUF(rp, r->sm, r->sc, xp, x->sm, x->sc, yp, y->sm, y->sc, C, l1, l2, l, N1, N2, offs); break; \
        case ORA_DIAG_BACK0: cell_diag_back0_##SUF(rp, r->sm, r->sc, xp, x->sm, x->sc, yp, y->sm, y->sc, C, l1, l2, l, N1, N2, offs); break; \
        case ORA_DIAG_BACK1: cell_diag_back1_##SUF(rp, r->sm, r->sc, xp, x->sm, x->sc, yp, y->sm, y->sc, C, l1, l2, l, N1, N2, offs); break; \
      }                                                                                                             \
    }                                                                                                               \
    free(C);                                                                                                        \
    return 0;                                                                                                       \
  }

DEFINE_CELL_KERNELS(float, f32)
DEFINE_CELL_KERNELS(double, f64)

/*
 * Part-level entry.  Roles are always (r, x, y) = (product or its gradient, first operand, second operand):
 * forward adds into r, back0 adds into x, back1 adds into y.  prec is 32 or 64.
 * Returns 0, or: 2 even m-dimension, 3 l outside the triangle, 4 Diag with N1!=N2, 5 offs+n_out exceeds r's
 * channels, 6 batch sizes cannot be reconciled.
 */
int ora_part_op(int op, int prec, const ora_part *r, const ora_part *x, const ora_part *y, int offs, int nthreads) {
  if (op < 0 || op > ORA_DIAG_BACK1) return 1;
  if (prec == 32) return part_op_f32(op, r, x, y, offs, nthreads);
  if (prec == 64) return part_op_f64(op, r, x, y, offs, nthreads);
  return 1;
}

/* ---- type arithmetic (core/Gtype.hpp:115-138) ---------------------------------------------------------------- */

/*
 * tau_out[l] for l = 0..ORA_MAXL*2, given the part lists (ascending l) of both operands.
 * maxl<0 keeps every l.  Returns the number of l with tau_out[l] > 0 ... the caller reads the array.
 */
int ora_type_product(int diag, int nx, const int *lx, const int *cx, int ny, const int *ly, const int *cy, int maxl,
                     int64_t *tau_out, int tau_len) {
  for (int i = 0; i < tau_len; i++) tau_out[i] = 0;
  int count = 0;
  for (int p = 0; p < nx; p++)
    for (int q = 0; q < ny; q++)
      for (int l = abs(lx[p] - ly[q]); l <= lx[p] + ly[q]; l++) {
        if (maxl >= 0 && l > maxl) continue;
        if (l >= tau_len) return -1;
        if (tau_out[l] == 0) count++;
        tau_out[l] += diag ? (int64_t)cx[p] : (int64_t)cx[p] * cy[q];
      }
  return count;
}

/* ---- vec-level entry (core/Gvec.hpp:311-389) ------------------------------------------------------------------
 * xparts, yparts, rparts: arrays of part descriptors, each list in ascending l (l read from M).
 * rparts is the product (forward) or its gradient (backward); parts of r that are absent are skipped
 * without advancing any other part's offset, exactly like the reference's per-l offset map.
 */
int ora_vec_op(int op, int prec, int nx, const ora_part *xparts, int ny, const ora_part *yparts, int nr,
               const ora_part *rparts, int nthreads) {
  int64_t offset[2 * ORA_MAXL + 2];
  for (int i = 0; i < 2 * ORA_MAXL + 2; i++) offset[i] = 0;
  int diag = (op >= ORA_DIAG_FWD);
  for (int p = 0; p < nx; p++) {
    for (int q = 0; q < ny; q++) {
      int l1 = (int)(xparts[p].M - 1) / 2, l2 = (int)(yparts[q].M - 1) / 2;
      for (int l = abs(l1 - l2); l <= l1 + l2; l++) {
        const ora_part *rp = NULL;
        for (int k = 0; k < nr; k++)
          if ((int)(rparts[k].M - 1) / 2 == l) rp = &rparts[k];
        if (!rp) continue;
        int rc = ora_part_op(op, prec, rp, &xparts[p], &yparts[q], (int)offset[l], nthreads);
        if (rc) return rc;
        offset[l] += diag ? xparts[p].N : xparts[p].N * yparts[q].N;
      }
    }
  }
  return 0;
}

/*
 * r[b, L+m, j] += Y_L^m(x[b,:,j] / |x[b,:,j]|) for every cell b and channel j (SO3/SO3part.hpp:340-403).
 * x is (B or 1, 3, n) float32 with strides (xsb, xsm, 1) in floats (xsb = 0 broadcasts one set of vectors over the
 * batch); r is (B, 2L+1, n) complex64, packed.  The arithmetic keeps the reference's types: the associated
 * Legendre table is float, each entry computed from a double expression; the phase runs in complex<float>.
 */
int ora_spharm(int L, long long B, long long n, const float *x, long long xsb, long long xsm, float *r) {
  if (L < 0 || L > ORA_MAXL) return 1;
  const int W = L + 1;
  float *P = (float *)malloc(sizeof(float) * (size_t)W * W);
  if (!P) return 1;
  for (long long b = 0; b < B; b++) {
    float *rb = r + 2 * b * (2 * L + 1) * n;
    const float *xb = x + b * xsb;
    for (long long j = 0; j < n; j++) {
      const float vx = xb[j], vy = xb[xsm + j], vz = xb[2 * xsm + j];
      const float length = sqrtf(vx * vx + vy * vy + vz * vz);
      const float len2 = sqrtf(vx * vx + vy * vy);
      if (len2 == 0 || isnan(vx / len2) || isnan(vy / len2)) {
        rb[2 * (L * n + j)] += (float)sqrt(((float)(2 * L + 1)) / (M_PI * 4.0));
        continue;
      }
      const float xx = vz / length;
      memset(P, 0, sizeof(float) * (size_t)W * W);
      P[0] = 1;
      const float xfact = (float)sqrt(1.0 - xx * xx);
      for (int l = 1; l <= L; l++) {
        P[l * W + l] = (float)(-(2.0 * l - 1.0) * xfact * P[(l - 1) * W + (l - 1)]);
        P[l * W + l - 1] = (float)((2.0 * l - 1.0) * P[(l - 1) * W + (l - 1)] * xx);
        for (int m = 0; m < l - 1; m++)
          P[l * W + m] = (float)(((2.0 * l - 1.0) * P[(l - 1) * W + m] * xx - ((float)(l + m - 1.0)) * (P[(l - 2) * W + m])) /
                                 ((float)(l - m)));
      }
      const float cr = vx / len2, ci = vy / len2;
      float pr = (float)sqrt((2.0 * L + 1.0) / (M_PI * 4.0)), pi = 0.f;
      for (int m = 0; m <= L; m++) {
        const float ar = pr * P[L * W + m], ai = pi * P[L * W + m];
        rb[2 * ((L + m) * n + j)] += ar;
        rb[2 * ((L + m) * n + j) + 1] += ai;
        if (m > 0) {
          const float sg = (float)(1 - 2 * (m % 2));
          rb[2 * ((L - m) * n + j)] += sg * ar;
          rb[2 * ((L - m) * n + j) + 1] += sg * (-ai);
        }
        if (m < L) {
          const float d = sqrtf((float)(L - m) * (L + m + 1));
          const float qr = cr / d, qi = ci / d;
          const float nr = pr * qr - pi * qi, ni = pr * qi + pi * qr;
          pr = nr;
          pi = ni;
        }
      }
    }
  }
  free(P);
  return 0;
}

int ora_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
