// SO3vec CGproduct followed by a channel-mixing matrix per product part, in one kernel: the product is never stored.
//
//   out_l[cell, m, o] (+)= sum_c P_l[cell, m, c] W_l[c, o],   P = CGproduct(x, y) (channels c in the reference's order)
//
// The mixing is a GEMM whose reduction runs over the product's channels; the product's element is its A operand and is
// computed by the lane that feeds it to the matrix cores.  v_mfma_f32_32x32x2_f32 computes D (32 x 32) += A (32 x 2)
// B (2 x 32); lane (i, h) = (lane % 32, lane / 32) supplies A[i][h] and B[h][i].  Here
//   rows of D   = 32 cells (one block = one wave = 32 cells), for one row (l, m) of the product;
//   the two k   = real and imaginary part of ONE product channel c: lane (i, h) computes component h of P_l[cell i, m, c]
//                 from its own cell's x and y -- only the component it needs;
//   columns     = (output channel, component): B[h][2 o + p] is the real 2 x 2 form of the complex W_l[c, o], re-packed
//                 once per call so that a wave's B operand of one channel is 256 contiguous bytes.
// Every (l, m) of the product needs its own 32 x 32 tile of sums (16 registers): l = 0..4 would be 25 tiles.  The rows
// are split by m into two passes, each a launch of its own: m < 0 with (m = 0, l >= 3) -- 12 tiles -- and m > 0 with
// (m = 0, l <= 2) -- 13 tiles, the same number of matrix instructions to within 1 %.  A product x[m1] y[m2] belongs to
// the one row m = m1 + m2, so apart from the nine of m = 0 every product is formed in one pass only.  Per channel pair
// (a, j) and row m the lane forms q(m1) = component h of x[m1, a] y[m - m1, j] (two operations each, shared by the l),
// then per l one multiply-add per term for P and one matrix instruction.  y of the current l2 sits in LDS transposed
// (consecutive cells side by side), x comes from a copy transposed the same way in global memory, one channel ahead,
// y one channel pair ahead, the B operands 3 to 15 channel pairs ahead (see wide_u).
//
// This header holds the kernel; cg_linear_pass0.hip and cg_linear_pass1.hip instantiate one launch each (the two
// compile side by side), cg_linear.hip holds the helper kernels and the host side.
#pragma once

#include "cg_diag6.h"
#include "cg_linear.h"
#include "cg_unrolled_dev.h"

namespace gelib_hip {

typedef float f16v __attribute__((ext_vector_type(16)));
typedef const __attribute__((address_space(4))) float *CoeffPtr;
typedef const __attribute__((address_space(1))) float *GlobalF;
typedef float v2f __attribute__((ext_vector_type(2)));
typedef const __attribute__((address_space(1))) v2f *GlobalC;

constexpr int kNL = kLinL + 1;

struct LinArgs {
  FastPart x[kNL], y[kNL], out[kNL];  // by l; operands: ptr == nullptr when the part is absent
  const float *wp[kNL];               // re-packed matrices by product l: 64 floats per product channel
  const float2 *xt[kNL];              // x by l, transposed per group of 32 cells: [group][row * n + channel][cell in group]
  int offs[kNL][kNL][kNL];            // [l1][l2][l]: first channel of the triple's block in product part l
  const float *bank;                  // coefficient tables, table_off(l1, l2, l)
  long long ncells;
  int accumulate;
};

constexpr int kBAhead = 16;  // most channel pairs between the load of a B operand and its use

// is row m of part l (|m| <= l) one of the pass?
constexpr bool in_pass(int pass, int l, int m) { return pass == 0 ? (m < 0 || (m == 0 && l >= 3)) : (m > 0 || (m == 0 && l <= 2)); }
// has the pass a row of part l at all?
constexpr bool l_in_pass(int pass, int l) { return pass == 0 ? l >= 1 : true; }
constexpr int tile_of(int pass, int l, int m) {
  if (m == 0) return pass == 0 ? 10 + (4 - l) : 10 + (2 - l);
  return l * (l - 1) / 2 + (m < 0 ? m + l : m - 1);
}
constexpr int kTiles = 13;

// does the pass have a row m of some l of the pair (l1, l2)?
constexpr bool row_needed(int pass, int l1, int l2, int m) {
  for (int l = iabs(l1 - l2); l <= imin(l1 + l2, kLinL); l++)
    if (iabs(m) <= l && in_pass(pass, l, m)) return true;
  return false;
}
// matrix instructions per channel pair that the pass issues for the pair (l1, l2): its rows (l, m)
constexpr int tile_count(int pass, int l1, int l2) {
  int n = 0;
  for (int l = iabs(l1 - l2); l <= imin(l1 + l2, kLinL); l++)
    for (int m = -l; m <= l; m++) n += in_pass(pass, l, m);
  return n;
}
// Channel pairs per trip of the inner loop = slots of the ring of B operands (at most 63 loads in flight: 5 l at most).  A slot is refilled right after its use,
// so a B operand is loaded U - 1 channel pairs ahead; the first wave of an XCD to touch a line of the matrices waits for
// memory beyond the L2 cache (a microsecond), and the waves of a launch walk the matrices together, so the load must be
// that far ahead in time: many channel pairs for the pairs that do little per channel pair.
constexpr int wide_u(int pass, int l1, int l2) {
  const int n = tile_count(pass, l1, l2);
  return n <= 2 ? 16 : (n <= 6 ? 8 : 4);
}
constexpr bool pair_needed(int pass, int l1, int l2) {
  for (int m = -kLinL; m <= kLinL; m++)
    if (row_needed(pass, l1, l2, m)) return true;
  return false;
}

template <int L1, int L2, int PASS, int U>
__device__ __forceinline__ void pair_body(const LinArgs &a, f16v (&acc)[kTiles], const v2f *ys, long long cell,
                                          int slot, int h, int lane, int zero) {
  constexpr int lmin = iabs(L1 - L2), lmax = imin(L1 + L2, kLinL);
  constexpr int R1 = 2 * L1 + 1, R2 = 2 * L2 + 1, NLP = lmax - lmin + 1;
  if constexpr (!pair_needed(PASS, L1, L2)) return;
  const FastPart X = a.x[L1];
  const int n1 = X.n, n2 = a.y[L2].n;
  // x from its transposed copy: the 32 cells of the block side by side, so a load touches two lines, not 32 (read from
  // the part itself -- eight bytes per cell, a cell's row apart -- the gathers of the waves of an XCD kept more lines
  // alive than its L2 cache holds and pushed the matrices out of it)
  const GlobalC xp = (GlobalC)(a.xt[L1] + (long long)blockIdx.x * (R1 * X.n) * kLinCells + slot);
  GlobalF wl[NLP];
  static_for<NLP>([&](auto dc) __attribute__((always_inline)) {
    constexpr int l = lmin + decltype(dc)::value;
    if constexpr (l_in_pass(PASS, l)) wl[dc.value] = (GlobalF)(a.wp[l] + (long long)a.offs[L1][L2][l] * 64 + lane);
  });

  // The coefficients of the pair's l of this pass, one register each (the same value in every lane): the scalar
  // registers cannot hold them all, and scalar loads inside the loop would each have to be waited for.  They are
  // fetched with VECTOR loads, all in flight at once: as scalar loads into one register each was loaded, waited for and
  // copied in turn (up to 97 round trips to the scalar cache per pair).  The lane offset `zero` is 0, but opaque to the
  // compiler, which would otherwise make scalar loads of them again.
  const GlobalF bankv = (GlobalF)a.bank + zero;
  float C[NLP][2 * (L1 + L2) + 1][R1];
  static_for<NLP>([&](auto dc) __attribute__((always_inline)) {
    constexpr int l = lmin + decltype(dc)::value;
    static_for<2 * l + 1>([&](auto mc) __attribute__((always_inline)) {
      constexpr int m = decltype(mc)::value - l;
      if constexpr (in_pass(PASS, l, m)) {
        static_for<R1>([&](auto kc) __attribute__((always_inline)) {
          constexpr int k = decltype(kc)::value, m2 = m - (k - L1);
          if constexpr (m2 >= -L2 && m2 <= L2) {
            C[dc.value][m + L1 + L2][k] = bankv[table_off(L1, L2, l) + k * R2 + (m2 + L2)];
          }
        });
      }
    });
  });

  // Channel pairs are taken U at a time so that the registers of operands in flight keep fixed names: the B operands
  // of the next U pairs sit in a ring of U slots (slot s is refilled, for the pair U further on, right after the matrix
  // instructions of sub-step s have read it), y alternates between two sets.  Copying a register that a load has
  // just been issued for would make the wave wait for that load.
  v2f xn[R1], yq[2][R2];
  float bq[U][NLP];
#pragma unroll
  for (int k = 0; k < R1; k++) xn[k] = xp[(k * n1) * kLinCells];
#pragma unroll
  for (int k = 0; k < R2; k++) yq[0][k] = ys[(k * n2) * kLinCells + slot];
  static_for<U>([&](auto ac) __attribute__((always_inline)) {
    static_for<NLP>([&](auto dc) __attribute__((always_inline)) {
      if constexpr (l_in_pass(PASS, lmin + decltype(dc)::value))
        bq[ac.value][dc.value] = wl[dc.value][ac.value * 64];
    });
  });

  int t = 0;  // channel of the block: a n2 + j
  for (int ia = 0; ia < n1; ia++) {
    // component h of x y is u yr + v yi with (u, v) = (xr, -xi) for the real part, (xi, xr) for the imaginary part
    float u[R1], v[R1];
#pragma unroll
    for (int k = 0; k < R1; k++) {
      u[k] = h ? xn[k].y : xn[k].x;
      v[k] = h ? xn[k].x : -xn[k].y;
    }
    const int ian = ia + 1 < n1 ? ia + 1 : ia;
#pragma unroll
    for (int k = 0; k < R1; k++) xn[k] = xp[(k * n1 + ian) * kLinCells];
    for (int j = 0; j < n2; j += U, t += U) {
      static_for<U>([&](auto sc) __attribute__((always_inline)) {
        constexpr int sub = decltype(sc)::value;
        constexpr int cur = U == 1 ? 0 : (sub & 1), nxt = U == 1 ? 1 : (cur ^ 1);
        // y of the next channel pair (first channel again behind the last: the next a)
        const int jn = j + sub + 1 < n2 ? j + sub + 1 : 0;
#pragma unroll
        for (int k = 0; k < R2; k++) yq[nxt][k] = ys[(k * n2 + jn) * kLinCells + slot];
        __builtin_amdgcn_sched_barrier(0);  // the loads stay ahead of the arithmetic that hides them (fences between the
                                            // rows, or in front of the refill below, cost 5 %: the chains of one row
                                            // depend on each other, and with one wave per SIMD nothing else fills in)

        static_for<2 * (L1 + L2) + 1>([&](auto mc) __attribute__((always_inline)) {
          constexpr int m = decltype(mc)::value - (L1 + L2);
          if constexpr (row_needed(PASS, L1, L2, m)) {
            float q[R1];
            static_for<R1>([&](auto kc) __attribute__((always_inline)) {
              constexpr int k = decltype(kc)::value, m2 = m - (k - L1);
              if constexpr (m2 >= -L2 && m2 <= L2)
                q[k] = __builtin_fmaf(v[k], yq[cur][m2 + L2].y, u[k] * yq[cur][m2 + L2].x);
            });
            static_for<NLP>([&](auto dc) __attribute__((always_inline)) {
              constexpr int l = lmin + decltype(dc)::value;
              if constexpr (iabs(m) <= l && in_pass(PASS, l, m)) {
                float P = 0.f;
                bool first = true;
                static_for<R1>([&](auto kc) __attribute__((always_inline)) {
                  constexpr int k = decltype(kc)::value, m2 = m - (k - L1);
                  if constexpr (m2 >= -L2 && m2 <= L2) {
                    const float c = C[dc.value][m + L1 + L2][k];
                    P = first ? c * q[k] : __builtin_fmaf(c, q[k], P);
                    first = false;
                  }
                });
                constexpr int tile = tile_of(PASS, l, m);
                acc[tile] = __builtin_amdgcn_mfma_f32_32x32x2f32(P, bq[sub][dc.value], acc[tile], 0, 0, 0);
              }
            });
          }
        });
        // refill the slot (the B operands past the block's last channel are the next block's or padding)
        static_for<NLP>([&](auto dc) __attribute__((always_inline)) {
          if constexpr (l_in_pass(PASS, lmin + decltype(dc)::value))
            bq[sub][dc.value] = wl[dc.value][(long long)(t + sub + U) * 64];
        });
        if constexpr (U == 1) {
#pragma unroll
          for (int k = 0; k < R2; k++) yq[0][k] = yq[1][k];
        }
      });
    }
  }
}

template <int PASS>
__global__ void __launch_bounds__(64) cg_linear_fwd_kernel(const LinArgs a) {
  __shared__ v2f ys[(2 * kLinL + 1) * kLinMaxN * kLinCells];
  const int lane = threadIdx.x, slot = lane & 31, h = lane >> 5;
  int zero;
  asm volatile("v_mov_b32 %0, 0" : "=v"(zero));
  const long long cell0 = (long long)blockIdx.x * kLinCells;
  long long cell = cell0 + slot;
  if (cell >= a.ncells) cell = a.ncells - 1;  // the last block's spare rows repeat the last cell and are not stored

  f16v acc[kTiles];
#pragma unroll
  for (int k = 0; k < kTiles; k++)
#pragma unroll
    for (int e = 0; e < 16; e++) acc[k][e] = 0.f;

  static_for<kNL>([&](auto l2c) __attribute__((always_inline)) {
    constexpr int L2 = decltype(l2c)::value;
    const FastPart Y = a.y[L2];
    if (Y.ptr != nullptr) {
      __syncthreads();
      const GlobalC yp = (GlobalC)(Y.ptr + cell * Y.sb);
      for (int row = 0; row < 2 * L2 + 1; row++)
        for (int j = h; j < Y.n; j += 2) ys[(row * Y.n + j) * kLinCells + slot] = yp[row * Y.sm + j];
      __syncthreads();
      static_for<kNL>([&](auto l1c) __attribute__((always_inline)) {
        constexpr int L1 = decltype(l1c)::value;
        if (a.x[L1].ptr != nullptr) {
          constexpr int UW = wide_u(PASS, L1, L2);
          // the second operand's channel count must be a multiple of the ring length; any other count takes one
          // channel pair per trip and waits for every load (correct, slow)
          if ((Y.n & (UW - 1)) == 0) pair_body<L1, L2, PASS, UW>(a, acc, ys, cell, slot, h, lane, zero);
          else pair_body<L1, L2, PASS, 1>(a, acc, ys, cell, slot, h, lane, zero);
        }
      });
    }
  });

  // register v of a tile: row (cell) 8 (v / 4) + 4 h + v % 4, column (float of the output row) = lane % 32
  static_for<kNL>([&](auto lc) __attribute__((always_inline)) {
    constexpr int l = decltype(lc)::value;
    const FastPart O = a.out[l];
    const int ncol = 2 * O.n;
    static_for<2 * l + 1>([&](auto rc) __attribute__((always_inline)) {
      constexpr int row = decltype(rc)::value;
      if constexpr (in_pass(PASS, l, row - l)) {
        constexpr int tile = tile_of(PASS, l, row - l);
#pragma unroll
        for (int v = 0; v < 16; v++) {
          const long long c = cell0 + 8 * (v / 4) + 4 * h + (v % 4);
          if (c < a.ncells && slot < ncol) {
            float *p = (float *)(O.ptr + c * O.sb + (long long)row * O.sm) + slot;
            *p = a.accumulate ? *p + acc[tile][v] : acc[tile][v];
          }
        }
      }
    });
  });
}

template <int PASS>
int launch_cg_linear_pass_impl(const LinArgs &a, long long nblocks, hipStream_t s) {
  cg_linear_fwd_kernel<PASS><<<dim3((unsigned)nblocks), dim3(64), 0, s>>>(a);
  GELIB_HIP_TRY(hipGetLastError());
  return GELIB_HIP_OK;
}

// one launch each, instantiated in cg_linear_pass0.hip / cg_linear_pass1.hip
int launch_cg_linear_pass0(const LinArgs &a, long long nblocks, hipStream_t s);
int launch_cg_linear_pass1(const LinArgs &a, long long nblocks, hipStream_t s);

}  // namespace gelib_hip
