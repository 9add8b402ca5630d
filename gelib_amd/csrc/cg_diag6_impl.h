// DiagCGproduct of SO3vecs whose parts have l <= 6 and more than 32 channels: forward, and both gradients from one
// pass over g, every loop over l1, l2, l, m unrolled at compile time.
//
// A Diag product pairs channel c of x with channel c of y, so nothing is ever summed across channels.  A wave takes
// one cell and 64 consecutive channels, lane = channel, and walks through all (l1,l2) pairs:
//   forward   P[m1,m2] = x[m1] y[m2] once per (m1,m2), then r_l[m1+m2] += C_l[m1,m2] P for every l of the pair; the rows
//             of one m are complete after its m1-loop and are stored as 512 contiguous bytes each;
//   backward  Q[m1,m2] = sum_l C_l[m1,m2] g_l[m1+m2], then ax[m1] += Q conj(y[m2]) and ay[m2] += Q conj(x[m1]).  The
//             x-gradient of part l1 stays in registers while l2 runs and is written once; the y-gradient is kept in
//             a wave-private image in LDS (49 rows of 64 lanes), each lane adding into its own column: no atomics, no
//             barrier, a fixed order of additions.
// The cell of a wave is uniform, so every row address is a scalar base plus the lane's channel: loads and stores use
// the scalar-base form and need no address arithmetic on the vector unit.  Coefficients of all (l1,l2,l) with
// l1, l2 <= 6 live in one table with compile-time offsets and are read with scalar loads.
#pragma once

#include "cg_diag6.h"
#include "cg_lane_sums.h"
#include "cg_unrolled_dev.h"

namespace gelib_hip {

namespace {

constexpr int kRowBudget = 28;        // rows of g a lane keeps in flight
constexpr int kRowBudgetPacked = 20;  // several cells per wave: a lane offset per part costs registers, and 168 is the limit

typedef float v2f __attribute__((ext_vector_type(2)));
typedef const __attribute__((address_space(1))) v2f *GlobalIn;
typedef __attribute__((address_space(1))) v2f *GlobalOut;
typedef const __attribute__((address_space(4))) float *CoeffPtr;
typedef const __attribute__((address_space(4))) int *OffsPtr;

// Rows are addressed as a wave-uniform byte pointer plus the lane's byte offset (32 bits, unsigned): the form the
// scalar-base load/store instructions take, so no address arithmetic runs on the vector unit.
typedef __attribute__((address_space(1))) char *RowPtr;

// (The empty asm keeps the widening of the offset next to its use; hoisted out of the block, the instruction selector
// no longer sees base + 32-bit offset and falls back to a 64-bit vector add per access.)
__device__ __forceinline__ float2 row_load(RowPtr row, unsigned lane_off) {
  asm volatile("" : "+v"(lane_off));
  const v2f t = *(GlobalIn)(row + lane_off);
  return make_float2(t.x, t.y);
}
__device__ __forceinline__ void row_store(RowPtr row, unsigned lane_off, float2 v, bool accumulate) {
  v2f o = {v.x, v.y};
  if (accumulate) {
    unsigned lo = lane_off;
    asm volatile("" : "+v"(lo));
    o += *(GlobalOut)(row + lo);
  }
  asm volatile("" : "+v"(lane_off));
  *(GlobalOut)(row + lane_off) = o;
}

// A wave covers 64 channels of one cell, or -- when a part has 32 channels or fewer -- all channels of 64 / n_pad
// consecutive cells (n_pad = the channel count rounded up to a power of two).  `cell` is the first cell of the wave and
// uniform; `cell_local` and `ch` are the lane's own.
struct WavePos {
  long long cell;
  int cell_local;
  int ch;     // a valid channel of a valid cell also for lanes that have nothing to do (they never store)
  bool live;
};

__device__ __forceinline__ WavePos wave_pos(const Diag6Args &a, long long w) {
  WavePos q;
  const int lane = (int)(threadIdx.x & 63);
  if (a.lg_npad < 6) {
    q.cell = w << (6 - a.lg_npad);
    q.cell_local = lane >> a.lg_npad;
    q.ch = lane & ((1 << a.lg_npad) - 1);
    q.live = q.ch < a.n && q.cell + q.cell_local < a.ncells;
  } else {
    q.cell = w / a.groups;
    q.cell_local = 0;
    q.ch = (int)(w - q.cell * a.groups) * 64 + lane;
    q.live = q.ch < a.n;
  }
  if (!q.live) q.cell_local = 0, q.ch = 0;
  return q;
}

// Byte offset of the lane's element from row 0 of the wave's first cell; 32 bits (the host checks the range).
// PACKED: several cells per wave, so the offset depends on the part's cell stride; otherwise it is the channel alone.
// bc: the part has ONE channel, which every lane reads (a CGproduct with a one-channel operand is the Diag product with
// that channel repeated); its gradient is then a sum over the lanes of a cell.
template <bool PACKED>
__device__ __forceinline__ unsigned lane_offset(const FastPart P, const WavePos q, bool bc = false) {
  const unsigned ch = bc ? 0u : (unsigned)q.ch;
  if constexpr (PACKED) return ((unsigned)q.cell_local * (unsigned)P.sb + ch) * 8u;
  else return ch * 8u;
}

// Row 0 of a part in the wave's cell, and the distance between its rows in bytes.
__device__ __forceinline__ RowPtr cell_row0(const FastPart P, long long cell) { return (RowPtr)P.ptr + cell * P.sb * 8; }
__device__ __forceinline__ long long row_step(const FastPart P) { return (long long)P.sm * 8; }

template <int L, bool PACKED>
__device__ __forceinline__ void load_rows(float2 (&v)[2 * L + 1], const FastPart P, const WavePos q, bool bc) {
  RowPtr row = cell_row0(P, q.cell);
  const long long step = row_step(P);
  const unsigned lo = lane_offset<PACKED>(P, q, bc);
#pragma unroll
  for (int m = 0; m <= 2 * L; m++) {
    v[m] = row_load(row, lo);
    row += step;
  }
}

// LLO: the launch takes only the l from LLO up (the part of a product above l = 6 is a launch of its own).
template <int L1, int L2, int LCAP, bool PACKED, int LLO = 0>
__device__ __forceinline__ void fwd_pair(const Diag6Args &a, const float2 (&xv)[2 * L1 + 1],
                                         const float2 (&yv)[2 * L2 + 1], const WavePos q) {
  constexpr int LMIN = imax(iabs(L1 - L2), LLO);
  constexpr int LTOP = imin(L1 + L2, LCAP);
  if constexpr (LMIN <= LTOP) {
    constexpr int NL = LTOP - LMIN + 1;
    const OffsPtr offs = (OffsPtr)a.offs + (L1 * kNP + L2) * kNR;
    const CoeffPtr C = (CoeffPtr)a.bank;
    const bool accumulate = a.accumulate != 0;
    // the row of part l that the next m of that part is stored to; a triple that is not there is never stored
    RowPtr row[NL];
    unsigned lo[NL];
    bool present[NL];
    static_for<NL>([&](auto dc) __attribute__((always_inline)) {
      constexpr int dl = decltype(dc)::value;
      const int off = offs[LMIN + dl];
      present[dl] = off >= 0;
      row[dl] = cell_row0(a.r[LMIN + dl], q.cell) + (long long)(off + a.offs_add) * 8;
      lo[dl] = lane_offset<PACKED>(a.r[LMIN + dl], q);
    });
    static_for<2 * LTOP + 1>([&](auto mc) __attribute__((always_inline)) {
      constexpr int m = decltype(mc)::value - LTOP;
      constexpr int MABS = iabs(m);
      constexpr int M1LO = imax(-L1, m - L2), M1HI = imin(L1, m + L2);
      float2 acc[NL];
#pragma unroll
      for (int k = 0; k < NL; k++) acc[k] = make_float2(0.f, 0.f);
      static_for<M1HI - M1LO + 1>([&](auto kc) __attribute__((always_inline)) {
        constexpr int m1 = M1LO + decltype(kc)::value;
        constexpr int m2 = m - m1;
        const float2 xa = xv[m1 + L1], yb = yv[m2 + L2];
        const float pr = fmaf(-xa.y, yb.y, xa.x * yb.x), pi = fmaf(xa.y, yb.x, xa.x * yb.y);
        static_for<NL>([&](auto dc) __attribute__((always_inline)) {
          constexpr int dl = decltype(dc)::value;
          constexpr int L = LMIN + dl;
          if constexpr (L >= MABS) {
            const float c = C[table_off(L1, L2, L) + (m1 + L1) * (2 * L2 + 1) + (m2 + L2)];
            acc[dl].x = fmaf(c, pr, acc[dl].x);
            acc[dl].y = fmaf(c, pi, acc[dl].y);
          }
        });
      });
      static_for<NL>([&](auto dc) __attribute__((always_inline)) {
        constexpr int dl = decltype(dc)::value;
        constexpr int L = LMIN + dl;
        if constexpr (L >= MABS) {
          if (present[dl] && q.live) row_store(row[dl], lo[dl], acc[dl], accumulate);
          row[dl] += row_step(a.r[L]);
        }
      });
    });
  }
}

// Copies the rows of all parts of one operand (the block's cell, or cells, and channel group) into LDS, row l*l + m of
// the image holding row m of part l, one column per lane.  The rows are dealt to the four waves in turn; every wave
// requests all of its rows before it writes the first one.
template <bool PACKED, int LOP>
__device__ __forceinline__ void stage_operand(float2 *img, const FastPart (&parts)[kNP], const WavePos q, int wave, int lane,
                                              bool bc) {
  constexpr int kRows = (LOP + 1) * (LOP + 1);  // rows of the parts l = 0..LOP
  constexpr int kPer = (kRows + 3) / 4;
  float2 v[kPer];
  static_for<kPer>([&](auto kc) __attribute__((always_inline)) {
    constexpr int k = decltype(kc)::value;
    const int r = 4 * k + wave;  // uniform for the wave
    v[k] = make_float2(0.f, 0.f);
    static_for<LOP + 1>([&](auto lc) __attribute__((always_inline)) {
      constexpr int L = decltype(lc)::value;
      if (r >= L * L && r < (L + 1) * (L + 1) && parts[L].ptr != nullptr)
        v[k] = row_load(cell_row0(parts[L], q.cell) + (long long)(r - L * L) * row_step(parts[L]), lane_offset<PACKED>(parts[L], q, bc));
    });
  });
  static_for<kPer>([&](auto kc) __attribute__((always_inline)) {
    constexpr int k = decltype(kc)::value;
    const int r = 4 * k + wave;
    if (r < kRows) img[r * 64 + lane] = v[k];
  });
}

template <int L>
__device__ __forceinline__ void read_rows(float2 (&v)[2 * L + 1], const float2 *img, int lane) {
#pragma unroll
  for (int m = 0; m <= 2 * L; m++) v[m] = img[(L * L + m) * 64 + lane];
}

// The four waves of a block work on the same cell and channel group and take every fourth pair: pairs that follow
// each other write neighbouring 512-byte blocks of the same product rows, so the rows fill in 2 KB at a time.
// The second operand of the block is copied to LDS first (25 KB): read straight from memory, the y part of each of
// the 49 pairs was fetched anew, seven times the operand in all, and a fetch in the middle of the store stream waits
// for the stores ahead of it.  x stays with the waves (every wave reads each part of it once): a second image would
// leave room for three blocks per compute unit instead of five, and the store stream needs the waves (measured on
// L = 6, 64 channels, 131072 cells: no image 18.2 - 20.2 ms, y alone 16.6 - 17.4 ms, both 29.7 ms).
// LOP: the largest l of an operand part the kernel has code for.
template <int LCAP, bool PACKED, int LOP, int LLO = 0>
__global__ void __launch_bounds__(256) diag6_fwd_kernel(const Diag6Args a) {
  __shared__ float2 yimg[(LOP + 1) * (LOP + 1) * 64];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const long long w = blockIdx.x;
  const WavePos q = wave_pos(a, w);
  stage_operand<PACKED, LOP>(yimg, a.y, q, wave, lane, a.ybc != 0);
  __syncthreads();
  static_for<LOP + 1>([&](auto l1c) __attribute__((always_inline)) {
    constexpr int L1 = decltype(l1c)::value;
    if constexpr (L1 + LOP >= LLO) {  // some pair of this l1 reaches an l the launch takes
      if (a.x[L1].ptr != nullptr) {
        float2 xv[2 * L1 + 1];
        load_rows<L1, PACKED>(xv, a.x[L1], q, a.xbc != 0);
        static_for<LOP + 1>([&](auto l2c) __attribute__((always_inline)) {
          constexpr int L2 = decltype(l2c)::value;
          if constexpr (L1 + L2 >= LLO) {
            if (((L1 * kNP + L2) & 3) == wave && a.y[L2].ptr != nullptr) {
              float2 yv[2 * L2 + 1];
              read_rows<L2>(yv, yimg, lane);
              fwd_pair<L1, L2, LCAP, PACKED, LLO>(a, xv, yv, q);
            }
          }
        });
      }
    }
  });
}

// One pair of the backward pass: every l of the pair together, one row number m = m1 + m2 at a time.
template <int L1, int L2, int LCAP, bool PACKED, int LLO = 0>
__device__ __forceinline__ void bwd_pair(const Diag6Args &a, const float2 (&xv)[2 * L1 + 1],
                                         const float2 (&yv)[2 * L2 + 1], float2 (&ax)[2 * L1 + 1], float2 *yimg,
                                         const WavePos q) {
  constexpr int LMIN = imax(iabs(L1 - L2), LLO);
  constexpr int LTOP = imin(L1 + L2, LCAP);
  if constexpr (LMIN <= LTOP) {
    constexpr int NL = LTOP - LMIN + 1;
    constexpr int ROWS = (LTOP + 1) * (LTOP + 1) - LMIN * LMIN;
    constexpr int kBudget = PACKED ? kRowBudgetPacked : kRowBudget;
    constexpr int PF = ROWS <= kBudget ? 2 * LTOP + 1 : (kBudget / NL > 1 ? kBudget / NL : 1);
    const OffsPtr offs = (OffsPtr)a.offs + (L1 * kNP + L2) * kNR;
    const CoeffPtr C = (CoeffPtr)a.bank;
    // a triple that is not there reads a row of zeros (its coefficients then do not matter), so the arithmetic has
    // no branches; row[dl] is the row of part l that the next m of that part is read from
    RowPtr row[NL];
    long long step[NL];
    unsigned lo[NL];
    static_for<NL>([&](auto dc) __attribute__((always_inline)) {
      constexpr int dl = decltype(dc)::value;
      constexpr int L = LMIN + dl;
      const int off = offs[L];
      const bool present = off >= 0;
      row[dl] = present ? cell_row0(a.r[L], q.cell) + (long long)(off + a.offs_add) * 8 : (RowPtr)(a.bank + kBankFloats);
      step[dl] = present ? row_step(a.r[L]) : 0;
      lo[dl] = present ? lane_offset<PACKED>(a.r[L], q) : (unsigned)q.ch * 8u;
    });
    float2 ay[2 * L2 + 1];
#pragma unroll
    for (int m2 = 0; m2 <= 2 * L2; m2++) ay[m2] = make_float2(0.f, 0.f);
    auto load_m = [&](auto mc, float2(&dst)[NL]) __attribute__((always_inline)) {
      constexpr int m = decltype(mc)::value - LTOP;
      static_for<NL>([&](auto dc) __attribute__((always_inline)) {
        constexpr int dl = decltype(dc)::value;
        if constexpr (LMIN + dl >= iabs(m)) {
          dst[dl] = row_load(row[dl], lo[dl]);
          row[dl] += step[dl];
        }
      });
    };
    float2 gq[PF][NL];
    static_for<PF>([&](auto kc) __attribute__((always_inline)) {
      if constexpr (kc.value <= 2 * LTOP) load_m(kc, gq[kc.value]);
    });
    static_for<2 * LTOP + 1>([&](auto mc) __attribute__((always_inline)) {
      constexpr int mi = decltype(mc)::value;
      constexpr int m = mi - LTOP;
      constexpr int MABS = iabs(m);
      float2 gl[NL];
#pragma unroll
      for (int k = 0; k < NL; k++) gl[k] = gq[mi % PF][k];
      if constexpr (mi + PF <= 2 * LTOP) load_m(std::integral_constant<int, mi + PF>{}, gq[mi % PF]);
      constexpr int M1LO = imax(-L1, m - L2), M1HI = imin(L1, m + L2);
      static_for<M1HI - M1LO + 1>([&](auto kc) __attribute__((always_inline)) {
        constexpr int m1 = M1LO + decltype(kc)::value;
        constexpr int m2 = m - m1;
        float qr = 0.f, qi = 0.f;
        static_for<NL>([&](auto dc) __attribute__((always_inline)) {
          constexpr int dl = decltype(dc)::value;
          constexpr int L = LMIN + dl;
          if constexpr (L >= MABS) {
            const float c = C[table_off(L1, L2, L) + (m1 + L1) * (2 * L2 + 1) + (m2 + L2)];
            qr = fmaf(c, gl[dl].x, qr);
            qi = fmaf(c, gl[dl].y, qi);
          }
        });
        const float2 yc = yv[m2 + L2], xc = xv[m1 + L1];
        ax[m1 + L1].x = fmaf(qr, yc.x, ax[m1 + L1].x);
        ax[m1 + L1].x = fmaf(qi, yc.y, ax[m1 + L1].x);
        ax[m1 + L1].y = fmaf(qi, yc.x, ax[m1 + L1].y);
        ax[m1 + L1].y = fmaf(-qr, yc.y, ax[m1 + L1].y);
        ay[m2 + L2].x = fmaf(qr, xc.x, ay[m2 + L2].x);
        ay[m2 + L2].x = fmaf(qi, xc.y, ay[m2 + L2].x);
        ay[m2 + L2].y = fmaf(qi, xc.x, ay[m2 + L2].y);
        ay[m2 + L2].y = fmaf(-qr, xc.y, ay[m2 + L2].y);
      });
      __builtin_amdgcn_sched_barrier(0);
    });
#pragma unroll
    for (int m1 = 0; m1 <= 2 * L1; m1++) asm volatile("" : "+v"(ax[m1].x), "+v"(ax[m1].y));
    float2 *col = yimg + (L2 * L2) * 64 + (threadIdx.x & 63);
#pragma unroll
    for (int m2 = 0; m2 <= 2 * L2; m2++) {
      float2 o = col[m2 * 64];
      o.x += ay[m2].x;
      o.y += ay[m2].y;
      col[m2 * 64] = o;
    }
  }
}

// bc: the part has one channel: the lanes' values are added over the lanes of a cell (2^lg_n of them, a fixed order of
// additions) and the cell's first lane stores the total.
template <int L, bool PACKED>
__device__ __forceinline__ void store_rows(const float2 *v, int vstride, const FastPart P, const WavePos q, bool accumulate,
                                           bool bc, int lg_n) {
  RowPtr row = cell_row0(P, q.cell);
  const long long step = row_step(P);
  const unsigned lo = lane_offset<PACKED>(P, q, bc);
  if (bc) {
    float2 t[2 * L + 1];
#pragma unroll
    for (int m = 0; m <= 2 * L; m++) t[m] = q.live ? v[m * vstride] : make_float2(0.f, 0.f);
    group_sum(t, 1 << lg_n);
    if (q.live && q.ch == 0) {
#pragma unroll
      for (int m = 0; m <= 2 * L; m++) {
        row_store(row, lo, t[m], accumulate);
        row += step;
      }
    }
    return;
  }
  if (!q.live) return;
#pragma unroll
  for (int m = 0; m <= 2 * L; m++) {
    row_store(row, lo, v[m * vstride], accumulate);
    row += step;
  }
}

// The four waves of a block share one cell and channel group.  Each owns the pairs of its set of l2 (a.owner[l2], dealt
// by the host so that the waves get about the same number of rows of y: {6}, {5,0}, {4,1}, {3,2} when every part up to
// l = 6 is there), so its rows of the y-gradient image are its own (plain read-add-write).  The x-gradient of part l1 gets a partial sum from every
// wave; the partials meet in LDS after the last pair of l1, are added in the order of the waves and written out, the
// rows dealt round-robin to the waves.  Pairs (l1, l2) and (l1, l2 +- 1) read neighbouring 512-byte blocks of the same
// rows of g, and they are in flight at about the same time.
// Three waves per SIMD (168 registers) is what the LDS of a block lets a compute unit hold; both forms fit by
// themselves (the packed one with a smaller row budget).  Forcing the limit with amdgpu_waves_per_eu instead changed the
// schedule for the worse (twice as many waits).
template <int LCAP, bool PACKED, int LOP, int LLO = 0>
__global__ void __launch_bounds__(256) diag6_bwd_kernel(const Diag6Args a) {
  constexpr int kXRows = 2 * LOP + 1;
  constexpr int kYRows = (LOP + 1) * (LOP + 1);
  __shared__ float2 yimg[kYRows * 64];
  __shared__ float2 xpart[4 * kXRows * 64];  // [wave][row][lane]
  const long long w = blockIdx.x;
  const WavePos q = wave_pos(a, w);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const bool accumulate = a.accumulate != 0;
  const bool wx = a.want_x != 0, wy = a.want_y != 0;
  for (int e = threadIdx.x; e < kYRows * 64; e += 256) yimg[e] = make_float2(0.f, 0.f);
  __syncthreads();
  static_for<LOP + 1>([&](auto l1c) __attribute__((always_inline)) {
    constexpr int L1 = decltype(l1c)::value;
    if constexpr (L1 + LOP < LLO) return;  // no pair of this l1 reaches an l the launch takes
    if (a.x[L1].ptr != nullptr) {  // the same for the whole block
      // x is needed for the y-gradient only and y for the x-gradient only; an operand whose gradient is not wanted is
      // never read (a part-level call for one gradient does not even have it) and enters as zeros
      float2 xv[2 * L1 + 1], ax[2 * L1 + 1];
      if (wy) {
        load_rows<L1, PACKED>(xv, a.x[L1], q, a.xbc != 0);
      } else {
#pragma unroll
        for (int m1 = 0; m1 <= 2 * L1; m1++) xv[m1] = make_float2(0.f, 0.f);
      }
#pragma unroll
      for (int m1 = 0; m1 <= 2 * L1; m1++) ax[m1] = make_float2(0.f, 0.f);
      static_for<LOP + 1>([&](auto l2c) __attribute__((always_inline)) {
        constexpr int L2 = LOP - decltype(l2c)::value;  // descending, so that neighbours in l2 run at the same time
        if constexpr (L1 + L2 >= LLO) {
          if (a.owner[L2] == wave && a.y[L2].ptr != nullptr) {
            float2 yv[2 * L2 + 1];
            if (wx) {
              load_rows<L2, PACKED>(yv, a.y[L2], q, a.ybc != 0);
            } else {
#pragma unroll
              for (int m2 = 0; m2 <= 2 * L2; m2++) yv[m2] = make_float2(0.f, 0.f);
            }
            bwd_pair<L1, L2, LCAP, PACKED, LLO>(a, xv, yv, ax, yimg, q);
          }
        }
      });
      if (!wx) return;  // continues with the next l1 (this is the body of a per-l1 lambda); uniform for the block
      float2 *mine = xpart + wave * kXRows * 64 + lane;
#pragma unroll
      for (int m1 = 0; m1 <= 2 * L1; m1++) mine[m1 * 64] = ax[m1];
      __syncthreads();
      const FastPart XG = a.xg[L1];
      RowPtr row0 = cell_row0(XG, q.cell);
      const long long step = row_step(XG);
      const bool xbc = a.xbc != 0;
      const unsigned xlo = lane_offset<PACKED>(XG, q, xbc);
      static_for<2 * L1 + 1>([&](auto rc) __attribute__((always_inline)) {
        constexpr int r = decltype(rc)::value;
        if ((r & 3) == wave) {  // uniform
          float2 t[1];
          t[0] = xpart[(0 * kXRows + r) * 64 + lane];
#pragma unroll
          for (int k = 1; k < 4; k++) {
            const float2 u = xpart[(k * kXRows + r) * 64 + lane];
            t[0].x += u.x;
            t[0].y += u.y;
          }
          if (xbc) {  // one channel of x: its gradient is the sum over the lanes of the cell
            if (!q.live) t[0] = make_float2(0.f, 0.f);
            group_sum(t, 1 << a.lg_npad);
            if (q.live && q.ch == 0) row_store(row0 + r * step, xlo, t[0], accumulate);
          } else if (q.live) {
            row_store(row0 + r * step, xlo, t[0], accumulate);
          }
        }
      });
      __syncthreads();
    }
  });
  static_for<LOP + 1>([&](auto l2c) __attribute__((always_inline)) {
    constexpr int L2 = decltype(l2c)::value;
    const FastPart YG = a.yg[L2];
    if constexpr (L2 + LOP >= LLO) {
      if (wy && a.owner[L2] == wave && YG.ptr != nullptr)
        store_rows<L2, PACKED>(yimg + (L2 * L2) * 64 + lane, 64, YG, q, accumulate, a.ybc != 0, a.lg_npad);
    }
  });
}

// The backward pass when every part of y up to l = 6 is there: the waves' sets of l2 are fixed at compile time, {6},
// {5, 0}, {4, 1}, {3, 2} (13, 12, 12, 12 rows), so a wave keeps its rows of y in registers from the first pair to the
// last and y is read once (the kernel above reads the rows of y[l2] again for every l1: 1.23 times the algorithmic
// bytes on L = 6, 64 channels).  Everything else is as above -- the y-gradient of a pair is added into the wave's rows
// of the image in LDS, the x-gradient partials meet in LDS after the last pair of an l1 -- so the sums are formed in
// the same order and the results are the same bits.  The four waves run four instantiations of the loop over l1 and
// meet at its two barriers per l1.
template <int LCAP, bool PACKED, int LA, int LB>
__device__ __forceinline__ void bwd_wave_set(const Diag6Args &a, float2 *yimg, float2 *xpart, const WavePos q, int wave,
                                             int lane) {
  constexpr int kXRows = 2 * kL6 + 1;
  constexpr int RB = LB >= 0 ? 2 * LB + 1 : 1;
  constexpr int LBX = LB >= 0 ? LB : 0;
  const bool accumulate = a.accumulate != 0;
  const bool wx = a.want_x != 0, wy = a.want_y != 0;
  float2 ya[2 * LA + 1], yb[RB];
#pragma unroll
  for (int m = 0; m <= 2 * LA; m++) ya[m] = make_float2(0.f, 0.f);
#pragma unroll
  for (int m = 0; m < RB; m++) yb[m] = make_float2(0.f, 0.f);
  if (wx) {
    load_rows<LA, PACKED>(ya, a.y[LA], q, a.ybc != 0);
    if constexpr (LB >= 0) load_rows<LBX, PACKED>(yb, a.y[LBX], q, a.ybc != 0);
  }
  static_for<kNP>([&](auto l1c) __attribute__((always_inline)) {
    constexpr int L1 = decltype(l1c)::value;
    if (a.x[L1].ptr != nullptr) {  // the same for the whole block
      float2 xv[2 * L1 + 1], ax[2 * L1 + 1];
      if (wy) {
        load_rows<L1, PACKED>(xv, a.x[L1], q, a.xbc != 0);
      } else {
#pragma unroll
        for (int m1 = 0; m1 <= 2 * L1; m1++) xv[m1] = make_float2(0.f, 0.f);
      }
#pragma unroll
      for (int m1 = 0; m1 <= 2 * L1; m1++) ax[m1] = make_float2(0.f, 0.f);
      bwd_pair<L1, LA, LCAP, PACKED>(a, xv, ya, ax, yimg, q);
      if constexpr (LB >= 0) bwd_pair<L1, LBX, LCAP, PACKED>(a, xv, yb, ax, yimg, q);
      if (!wx) return;  // continues with the next l1; uniform for the block
      float2 *mine = xpart + wave * kXRows * 64 + lane;
#pragma unroll
      for (int m1 = 0; m1 <= 2 * L1; m1++) mine[m1 * 64] = ax[m1];
      __syncthreads();
      const FastPart XG = a.xg[L1];
      RowPtr row0 = cell_row0(XG, q.cell);
      const long long step = row_step(XG);
      const bool xbc = a.xbc != 0;
      const unsigned xlo = lane_offset<PACKED>(XG, q, xbc);
      static_for<2 * L1 + 1>([&](auto rc) __attribute__((always_inline)) {
        constexpr int r = decltype(rc)::value;
        if ((r & 3) == wave) {  // uniform
          float2 t[1];
          t[0] = xpart[(0 * kXRows + r) * 64 + lane];
#pragma unroll
          for (int k = 1; k < 4; k++) {
            const float2 u = xpart[(k * kXRows + r) * 64 + lane];
            t[0].x += u.x;
            t[0].y += u.y;
          }
          if (xbc) {  // one channel of x: its gradient is the sum over the lanes of the cell
            if (!q.live) t[0] = make_float2(0.f, 0.f);
            group_sum(t, 1 << a.lg_npad);
            if (q.live && q.ch == 0) row_store(row0 + r * step, xlo, t[0], accumulate);
          } else if (q.live) {
            row_store(row0 + r * step, xlo, t[0], accumulate);
          }
        }
      });
      __syncthreads();
    }
  });
  if (wy) {
    if (a.yg[LA].ptr != nullptr)
      store_rows<LA, PACKED>(yimg + (LA * LA) * 64 + lane, 64, a.yg[LA], q, accumulate, a.ybc != 0, a.lg_npad);
    if constexpr (LB >= 0)
      if (a.yg[LBX].ptr != nullptr)
        store_rows<LBX, PACKED>(yimg + (LBX * LBX) * 64 + lane, 64, a.yg[LBX], q, accumulate, a.ybc != 0, a.lg_npad);
  }
}

template <int LCAP, bool PACKED>
__global__ void __launch_bounds__(256) diag6_bwd_sets_kernel(const Diag6Args a) {
  __shared__ float2 yimg[kImgRows * 64];
  __shared__ float2 xpart[4 * (2 * kL6 + 1) * 64];  // [wave][row][lane]
  const WavePos q = wave_pos(a, blockIdx.x);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  for (int e = threadIdx.x; e < kImgRows * 64; e += 256) yimg[e] = make_float2(0.f, 0.f);
  __syncthreads();
  if (wave == 0) bwd_wave_set<LCAP, PACKED, 6, -1>(a, yimg, xpart, q, wave, lane);
  else if (wave == 1) bwd_wave_set<LCAP, PACKED, 5, 0>(a, yimg, xpart, q, wave, lane);
  else if (wave == 2) bwd_wave_set<LCAP, PACKED, 4, 1>(a, yimg, xpart, q, wave, lane);
  else bwd_wave_set<LCAP, PACKED, 3, 2>(a, yimg, xpart, q, wave, lane);
}

template <int LCAP, bool PACKED>
int launch_diag6_bwd_sets_variant(const Diag6Args &a, hipStream_t s) {
  hipLaunchKernelGGL((diag6_bwd_sets_kernel<LCAP, PACKED>), dim3((unsigned)a.nwaves), dim3(256), 0, s, a);
  GELIB_HIP_TRY(hipGetLastError());
  return GELIB_HIP_OK;
}

template <int LCAP, bool PACKED, int LOP = kL6, int LLO = 0>
int launch_diag6_fwd_variant(const Diag6Args &a, hipStream_t s) {
  hipLaunchKernelGGL((diag6_fwd_kernel<LCAP, PACKED, LOP, LLO>), dim3((unsigned)a.nwaves), dim3(256), 0, s, a);
  GELIB_HIP_TRY(hipGetLastError());
  return GELIB_HIP_OK;
}

template <int LCAP, bool PACKED, int LOP = kL6, int LLO = 0>
int launch_diag6_bwd_variant(const Diag6Args &a, hipStream_t s) {
  hipLaunchKernelGGL((diag6_bwd_kernel<LCAP, PACKED, LOP, LLO>), dim3((unsigned)a.nwaves), dim3(256), 0, s, a);
  GELIB_HIP_TRY(hipGetLastError());
  return GELIB_HIP_OK;
}

}  // namespace

}  // namespace gelib_hip
