// Backward pass of a product of ONE x part with ONE y part of large l on the matrix cores: both gradients from one pass
// over g (the l1 = l2 = 10, all 21 l case; any l1 <= 15, l2 <= 15, at most 22 values of l).  Described for 8 x 8
// channels, one wave per cell; PairShape below says how the other channel counts map onto the same scheme (16 channels:
// one tile instead of four; 128 or 256 channels: two or four waves per cell, 64 channels each).
//
// For one row number m = m1 + m2 the contraction over l,
//     Q[m1, chan] = sum_l C_l[m1, m - m1] g_l[m, chan],
// is a real (m1 x l) matrix times the (l x 128) block of the floats of the rows g_l[m] -- GEMM-shaped, with up to 21 x 21
// coefficients per m.  v_mfma_f32_32x32x2_f32 computes D (32 x 32) += A (32 x 2) B (2 x 32): here the rows of D are the
// floats of the 64 channels (four tiles of 32), its columns are m1, a step of the reduction is two values of l.
//   A: lane (i, h) = (lane % 32, lane / 32) loads 16 bytes of row g_{l(h)}[m], floats 4 i .. 4 i + 3, one for each of the
//      four tiles: a wave's load instruction fetches the two rows of a step, 512 contiguous bytes each;
//   B: lane (i, h) supplies C_{l(h)}[m1 = i - l1, m - m1], from a table laid out in lane order (one float per lane, step
//      and m), zero where the pair (m1, m2) or the value of l does not exist;
//   D: lane (i, h) ends up with Q[m1 = i - l1] of the 32 channels (a, j) with a = 2 b + h, b = 0..3, j = 0..7, real and
//      imaginary part: register v of tile e is float 4 (8 (v / 4) + 4 h + v % 4) + e of the row.
// So after the matrix instructions of one m a lane owns ONE m1 and with it one m2 = m - m1:
//   x-gradient  ax[m1, a] += sum_j Q[a, j] conj(y[m2, j]): the lane's m1 never changes, the sums are eight registers;
//   y-gradient  the lane's partial sum for ay[m2, j] (over its four a) belongs to a row m2 that moves on by one lane when
//               m goes up by one.  The eight partial sums travel with it: after every m they are shifted one lane up
//               (wave_shr), zeros enter at m1 = -l1, and the row that has left m1 = l1 is complete and is parked in LDS.
// No atomics, a fixed order of additions.  The vector unit does 256 multiply-adds per m and lane (both gradients),
// the matrix cores the 2 x (21 - |m|)^2 x 128 of the contraction; the operands of the next eight steps are always in
// flight, across the boundaries between the m.
//
// The forward pass of the same product (second kernel of this file) is the mirror image: for one m
//     r_l[m, chan] = sum_m1 P_m[chan, m1] C_l[m1, m - m1],   P_m[chan, m1] = x[m1, a] y[m - m1, j],
// here the ROWS of D are the l and its columns the floats of the 64 channels (four tiles of 32 columns), a step of the
// reduction is two values of m1.  Lane (i, h) supplies C_{lmin + i}[m1(h), m - m1(h)] from a table in lane order (the A
// operand) and forms four floats of the product x[m1(h)] y[m - m1(h)] from LDS (the B operands of the four tiles): column
// i of tile t is float 4 i + t of the row, i.e. the lane's floats are the real and imaginary parts of channels 2 i and
// 2 i + 1 = (a, j) and (a, j + 1) with a = i / 4: one x, two neighbouring y, eight operations.  After the steps of one m
// register v of the four tiles holds floats 4 i .. 4 i + 3 of row r_l[m] with l = lmin + 8 (v / 4) + 4 h + v % 4: one
// 16-byte store per lane, and a store instruction writes one complete 512-byte row for each half of the wave.  (With
// the channels as rows and the l as columns a lane owned 16-byte pieces of 21 different rows and the stores left as
// 32-byte pieces: 1.47 ms instead of the any-l kernel's 1.05.)
#include <cstring>
#include <map>
#include <type_traits>
#include <mutex>
#include <vector>

#include "cg_staged.h"
#include "cg_unrolled_dev.h"

namespace gelib_hip {

namespace {

constexpr int kNLm = 22;   // most values of l of the pair
constexpr int kMaxLm = 15; // largest l1, l2: 2 l + 1 <= 31 columns, one spare for the row that leaves

struct OnePairMfmaArgs {
  FastPart x, y, xg, yg;
  FastPart g[kNLm];   // by dl = l - lmin; ptr == nullptr: no such triple
  int offs[kNLm];     // first channel of the triple's block in its part
  const float *coef;  // device: 64 floats (lane order) per (m, step)
  int nsteps;         // steps of all m, rounded up to a multiple of the kernel's queue length (idle steps at the end)
  const float *coef_fwd;  // the same for the forward kernel (steps over m1, columns l)
  int nsteps_fwd;
  long long rowb;         // forward: bytes between the rows of every part of the product
  long long ncells;
  int l1, l2, lmin, lt, nl;
  int offs_add, accumulate;
  int paired;  // backward: the row numbers run in pairs (m, m + 2 l1 + 1), see the kernel
};

typedef float f16v __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef const __attribute__((address_space(1))) v4f *GlobalIn4;
typedef __attribute__((address_space(1))) v4f *GlobalOut4;
typedef const __attribute__((address_space(1))) float *GlobalIn1;
typedef __attribute__((address_space(1))) float *GlobalOut1;
typedef const __attribute__((address_space(4))) int *IntPtr;

__device__ __forceinline__ float wave_shr1(float v) {  // lane k receives lane k - 1, lane 0 receives 0
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x138, 0xf, 0xf, true));
}

constexpr int kQueue = 6;  // steps whose operands are in flight or waiting in registers

// How the N1 x N2 channels (a, j) of a block, channel a N2 + j, meet the matrix tiles.  A wave takes 64 neighbouring
// channels, four tiles of 32 floats (lane i loads floats 4 i .. 4 i + 3 of its piece of a row, one float per tile), or
// all 16 channels, one tile (lane i loads float i).  Register v of the tiles of lane (i, h) then holds channel
//     (CW / 4) (v / 4) + (CW / 8) h + jj,   jj = 0 .. JL - 1,
// of the wave's CW channels (four tiles: jj = 2 (v % 4) + e / 2, real part in tile e even, imaginary part in tile e + 1;
// one tile: jj = (v % 4) / 2, real part in v even, imaginary part in v + 1).  If the lane's JL channels are a whole row of
// j (JL = N2), the two halves of the wave hold different a (a = 2 (v / 4) + h): a lane's x-gradient sums are complete,
// the y-gradient is added over the halves.  Otherwise (2 JL = N2) the halves hold different j (j = JL h + jj,
// a = v / 4): the y-gradient sums of the wave are complete, the x-gradient is added over the halves.  Several waves:
// wave w has the channels a = w CW / N2 .. of x, and the y-gradient is added over the waves at the end.
template <int N1, int N2>
struct PairShape {
  static constexpr int kChan = N1 * N2;
  static constexpr int T = kChan >= 64 ? 4 : 1;
  static constexpr int W = kChan >= 64 ? kChan / 64 : 1;
  static constexpr int CW = 16 * T;
  static constexpr int JL = T == 4 ? 8 : 2;
  static constexpr bool kHalfIsA = JL == N2;
  static constexpr int kSlots = kHalfIsA ? 2 : 1;  // images of the y-gradient a wave parks its rows in
  static constexpr int kAWave = CW / N2;           // channels a of a wave
  static_assert(kChan == 16 || kChan % 64 == 0, "16 channels, or whole waves of 64");
  static_assert(W >= 1 && W <= 4, "at most four waves per cell");
  static_assert(JL == N2 || 2 * JL == N2, "a lane holds a whole row of j or half of one");
};

template <int N1, int N2>
__global__ void __launch_bounds__((64 * PairShape<N1, N2>::W)) onepair_mfma_bwd_kernel(const OnePairMfmaArgs a) {
  using Sh = PairShape<N1, N2>;
  constexpr int T = Sh::T, JL = Sh::JL, W = Sh::W;
  constexpr bool kHalfIsA = Sh::kHalfIsA;
  using GT = std::conditional_t<T == 4, v4f, float>;
  __shared__ unsigned long long gbase[kNLm + 1];  // address of row 0 of the cell's block in part dl; slot nl: a harmless row
  __shared__ unsigned growb[kNLm + 1];            // distance between rows in bytes
  __shared__ float2 ys[(2 * kMaxLm + 1) * N2];
  __shared__ float2 accy_all[W * Sh::kSlots][(2 * kMaxLm + 1) * N2];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63, i = lane & 31, h = lane >> 5;
  float2(*accy)[(2 * kMaxLm + 1) * N2] = accy_all + wave * Sh::kSlots;
  const int jbase = kHalfIsA ? 0 : JL * h;  // the lane's first channel j
  // channel a of the sums q = 0..3 of the lane
  auto a_of = [&](int q) __attribute__((always_inline)) { return wave * Sh::kAWave + (kHalfIsA ? 2 * q + h : q); };
  const int l1 = a.l1, l2 = a.l2, lmin = a.lmin, lt = a.lt, nl = a.nl;
  const long long cell = blockIdx.x;
  const int r1 = 2 * l1 + 1, r2 = 2 * l2 + 1;

  static_for<kNLm>([&](auto dc) __attribute__((always_inline)) {
    constexpr int dl = decltype(dc)::value;
    if (threadIdx.x == 0 && dl < nl) {
      const FastPart P = a.g[dl];
      const bool there = P.ptr != nullptr;
      // a triple that is not there reads the coefficient table (finite numbers) and meets coefficients that are zero
      gbase[dl] = there ? (unsigned long long)(P.ptr + cell * P.sb + (a.offs[dl] + a.offs_add)) : (unsigned long long)a.coef;
      growb[dl] = there ? (unsigned)P.sm * 8u : 0u;
    }
  });
  if (threadIdx.x == 0) {
    gbase[nl] = (unsigned long long)a.coef;
    growb[nl] = 0u;
  }
  for (int e = threadIdx.x; e < r2 * N2; e += 64 * W) {
    ys[e] = a.y.ptr[cell * a.y.sb + (long long)(e / N2) * a.y.sm + (e % N2)];
#pragma unroll
    for (int k = 0; k < W * Sh::kSlots; k++) accy_all[k][e] = make_float2(0.f, 0.f);
  }
  // the lane's row of x: m1 = i - l1, its four channels a; a lane beyond the rows holds zeros (so do its coefficients)
  float2 xv[4];
#pragma unroll
  for (int b = 0; b < 4; b++)
    xv[b] = i < r1 ? a.x.ptr[cell * a.x.sb + (long long)i * a.x.sm + a_of(b)] : make_float2(0.f, 0.f);
  __syncthreads();

  // The steps of all m form one sequence (two values of l per step, m ascending), padded with idle steps to a multiple
  // of kQueue.  The operands of the next kQueue steps are always on their way: a step's registers are refilled for the
  // step kQueue further on as soon as its matrix instructions are issued.  No load sits behind a branch.
  const int nsteps = a.nsteps;
  // where a step stands: its m, the first of its two dl, and how many steps of this m are left (itself included);
  // scalar arithmetic only.  Beyond the last m the cursor idles on the harmless row.
  struct Cursor {
    int m, dlb, left;
  };
  auto start_m = [&](Cursor &c, int m) __attribute__((always_inline)) {
    const int mabs = m < 0 ? -m : m;
    const int dl0 = (mabs > lmin ? mabs : lmin) - lmin;  // the first l with a row m
    c.m = m;
    c.dlb = dl0;
    c.left = (nl - dl0 + 1) >> 1;
  };
  // Order of the row numbers.  Plain: -lt .. lt.  Paired (l1 = l2, every l up to 2 l1 possible): -lt, 1, -lt + 1, 2,
  // ..., -1, lt, 0.  For m < 0 the pairs (m1, m2) with m1 + m2 = m occupy the columns m1 = -l1 .. m + l2, for
  // m' = m + 2 l1 + 1 > 0 the columns m1 = m' - l2 .. l1 = m + l1 + 1 .. l1: the two sets are complementary, and the
  // coefficient of a column that has no pair for the row number of a step is zero.  So the matrix steps of m and of m'
  // add into ONE set of sums (different columns), and the vector work that follows the matrix steps -- the same number
  // of instructions whether 1 or 21 columns hold a pair -- runs 21 times instead of 41.  A column's row of y moves on by one
  // per pair of row numbers exactly as it does per row number, so the sums of the y-gradient travel as before; a row
  // of the y-gradient now collects its terms with m > 0 first (parked when it leaves the last column) and those with
  // m <= 0 afterwards (added at the end).
  const int paired = a.paired;
  auto is_last = [&](int m) __attribute__((always_inline)) { return paired ? m == 0 : m == lt; };
  auto closes = [&](int m) __attribute__((always_inline)) { return !paired || m >= 0; };  // the sums are complete after m
  auto next_step = [&](Cursor &c) __attribute__((always_inline)) {
    if (--c.left > 0) {
      c.dlb += 2;
    } else if (!is_last(c.m)) {
      start_m(c, paired ? (c.m < 0 ? c.m + 2 * l1 + 1 : c.m - 2 * l1) : c.m + 1);
    } else {
      c.dlb = nl;
      c.left = 1 << 30;
    }
  };
  GT G[kQueue];
  float C[kQueue];
  long long coef_at = lane;  // the lane's coefficient of the step that is fetched next
  // the lane's piece of a row: 4 T bytes, 512 bytes on for every wave; the harmless row (the coefficient table) is
  // read at the same offsets, which its idle steps at the end cover
  const unsigned lane_off = (unsigned)wave * 512u + (unsigned)i * (4u * T);
  auto fetch = [&](const Cursor &c, GT &g, float &cf) __attribute__((always_inline)) {
    int dl = c.dlb + h;
    dl = dl < nl ? dl : nl;
    const unsigned long long base = gbase[dl];
    const unsigned rowb = growb[dl];
    const unsigned long long addr = base + (unsigned long long)((unsigned)(c.m + lmin + dl) * rowb) + lane_off;
    if constexpr (T == 4) g = *(GlobalIn4)addr;
    else g = *(GlobalIn1)addr;
    cf = *((GlobalIn1)a.coef + coef_at);   // the table ends with a queue's worth of idle steps
    coef_at += 64;
  };

  float2 ax[4], S[JL];
#pragma unroll
  for (int b = 0; b < 4; b++) ax[b] = make_float2(0.f, 0.f);
#pragma unroll
  for (int j = 0; j < JL; j++) S[j] = make_float2(0.f, 0.f);
  f16v D[T];

  // the sums of one m are in D: both gradients, then every row of the y-gradient moves one lane up
  auto finish_m = [&](int m) __attribute__((always_inline)) {
    // the lane's m2 = m - m1; outside [-l2, l2] (or m1 beyond l1) every coefficient was zero and so is Q.  Paired: the
    // columns up to m1 = mneg + l2 belong to the negative row number of the pair
    const int mneg = m - 2 * l1 - 1;
    const int mlane = (paired && m > 0 && (i - l1) <= mneg + l2) ? mneg : m;
    int m2 = mlane - (i - l1);
    m2 = m2 < -l2 ? -l2 : (m2 > l2 ? l2 : m2);
    const float4 *yrow = reinterpret_cast<const float4 *>(ys + (m2 + l2) * N2 + jbase);
    float2 yv[JL];
#pragma unroll
    for (int q = 0; q < JL / 2; q++) {
      const float4 t = yrow[q];
      yv[2 * q] = make_float2(t.x, t.y);
      yv[2 * q + 1] = make_float2(t.z, t.w);
    }
#pragma unroll
    for (int b = 0; b < 4; b++)
#pragma unroll
      for (int j = 0; j < JL; j++) {
        float qr, qi;
        if constexpr (T == 4) {
          qr = D[2 * (j & 1)][4 * b + (j >> 1)];
          qi = D[2 * (j & 1) + 1][4 * b + (j >> 1)];
        } else {
          qr = D[0][4 * b + 2 * j];
          qi = D[0][4 * b + 2 * j + 1];
        }
        ax[b].x = fmaf(qr, yv[j].x, ax[b].x);
        ax[b].x = fmaf(qi, yv[j].y, ax[b].x);
        ax[b].y = fmaf(qi, yv[j].x, ax[b].y);
        ax[b].y = fmaf(-qr, yv[j].y, ax[b].y);
        S[j].x = fmaf(qr, xv[b].x, S[j].x);
        S[j].x = fmaf(qi, xv[b].y, S[j].x);
        S[j].y = fmaf(qi, xv[b].x, S[j].y);
        S[j].y = fmaf(-qr, xv[b].y, S[j].y);
      }
    if (!is_last(m)) {  // the row that leaves m1 = l1 is complete (paired: its terms with m > 0 are); after the last m the rows stay where they are
#pragma unroll
      for (int j = 0; j < JL; j++) {
        S[j].x = wave_shr1(S[j].x);
        S[j].y = wave_shr1(S[j].y);
      }
      const int mdone = m - l1;  // the row now in column r1
      if (i == r1 && mdone >= -l2 && mdone <= l2) {
        float4 *dst = reinterpret_cast<float4 *>(accy[kHalfIsA ? h : 0] + (mdone + l2) * N2 + jbase);
#pragma unroll
        for (int q = 0; q < JL / 2; q++) dst[q] = make_float4(S[2 * q].x, S[2 * q].y, S[2 * q + 1].x, S[2 * q + 1].y);
      }
      if (i == 0 || i >= r1) {  // zeros enter at m1 = -l1; nothing travels on beyond the last column
#pragma unroll
        for (int j = 0; j < JL; j++) S[j] = make_float2(0.f, 0.f);
      }
    }
  };

  // The fences keep the loads in the order of the steps, here as in the loop: the wait in front of a step's matrix
  // instructions then counts the loads issued after its own instead of waiting for all.
  Cursor cf, ck;
  start_m(cf, -lt);
  start_m(ck, -lt);
  static_for<kQueue>([&](auto kc) __attribute__((always_inline)) {
    fetch(cf, G[kc.value], C[kc.value]);
    next_step(cf);
    __builtin_amdgcn_sched_barrier(0);
  });
  bool fresh = true;
  for (int q0 = 0; q0 < nsteps; q0 += kQueue) {
    static_for<kQueue>([&](auto kc) __attribute__((always_inline)) {
      constexpr int k = decltype(kc)::value;
      const GT g = G[k];
      const float c = C[k];
      auto piece = [&](int e) __attribute__((always_inline)) {
        if constexpr (T == 4) return g[e];
        else return g;
      };
      if (fresh) {  // uniform: the first step of an m starts from zero (a constant operand, no registers to clear)
        f16v zero;
#pragma unroll
        for (int v = 0; v < 16; v++) zero[v] = 0.f;
#pragma unroll
        for (int e = 0; e < T; e++) D[e] = __builtin_amdgcn_mfma_f32_32x32x2f32(piece(e), c, zero, 0, 0, 0);
      } else {
#pragma unroll
        for (int e = 0; e < T; e++) D[e] = __builtin_amdgcn_mfma_f32_32x32x2f32(piece(e), c, D[e], 0, 0, 0);
      }
      fresh = ck.left == 1 && closes(ck.m);  // the next step starts new sums
      fetch(cf, G[k], C[k]);
      next_step(cf);
      __builtin_amdgcn_sched_barrier(0);
      if (ck.left == 1 && closes(ck.m)) finish_m(ck.m);  // uniform; an idle step never ends an m
      next_step(ck);
    });
  }
  // the rows that are still on their way are complete as well: column i holds m2 = (the last m) - (i - l1).  They are
  // added to what is parked (zeros, or -- paired -- the row's terms with m > 0)
  {
    const int m2 = (paired ? 0 : lt) - (i - l1);
    if (i < r1 && m2 >= -l2 && m2 <= l2) {
      float4 *dst = reinterpret_cast<float4 *>(accy[kHalfIsA ? h : 0] + (m2 + l2) * N2 + jbase);
#pragma unroll
      for (int q = 0; q < JL / 2; q++) {
        const float4 o = dst[q];
        dst[q] = make_float4(o.x + S[2 * q].x, o.y + S[2 * q].y, o.z + S[2 * q + 1].x, o.w + S[2 * q + 1].y);
      }
    }
  }
  __syncthreads();

  const bool accumulate = a.accumulate != 0;
  if constexpr (!kHalfIsA) {  // the two halves of the wave hold the sums over different j
#pragma unroll
    for (int b = 0; b < 4; b++) {
      ax[b].x += __shfl_xor(ax[b].x, 32);
      ax[b].y += __shfl_xor(ax[b].y, 32);
    }
  }
  if (i < r1) {
#pragma unroll
    for (int b = 0; b < 4; b++) {
      if (!kHalfIsA && (b >> 1) != h) continue;  // each half stores two of the four
      float2 *p = a.xg.ptr + cell * a.xg.sb + (long long)i * a.xg.sm + a_of(b);
      float2 o = ax[b];
      if (accumulate) o.x += p->x, o.y += p->y;
      *p = o;
    }
  }
  for (int e = threadIdx.x; e < r2 * N2; e += 64 * W) {
    float2 *p = a.yg.ptr + cell * a.yg.sb + (long long)(e / N2) * a.yg.sm + (e % N2);
    float2 o = accy_all[0][e];
#pragma unroll
    for (int k = 1; k < W * Sh::kSlots; k++) o.x += accy_all[k][e].x, o.y += accy_all[k][e].y;
    if (accumulate) o.x += p->x, o.y += p->y;
    *p = o;
  }
}


constexpr int kStepsM = (2 * kMaxLm + 2) / 2;  // most steps of one m (forward): two values of m1 per step
constexpr int kColsF = 24;                     // columns (values of l) the forward coefficient table keeps per step and m1
constexpr int kCellsF = 8;                     // cells (waves) per block of the forward kernel

// Forward: g[] are the parts of the product (written), x and y the operands.  A block of eight waves takes eight cells
// (four or two when a cell's 128 or 256 channels take two or four waves) and shares one copy of the coefficient table
// in LDS (2 x 24 floats per step, 44 KB at l1 = l2 = 10), loaded by all of its threads while the waves set up their
// cells.  Nothing is loaded from memory once the rows are being stored: loads and stores return through one in-order
// counter, and a wait for a load issued behind stores waits for the stores to be acknowledged (with the coefficients
// fetched from memory step by step the waves spent a third of their time so).
// ONE_ROWB: all parts have the same row length a.rowb (true whenever the parts hold just this pair's block); otherwise
// every register row carries its own.
// Channels: a wave's columns are the floats of 64 neighbouring channels (column i of tile t = float 4 i + t: the lane
// forms the products of channels 2 i and 2 i + 1 = (a, j) and (a, j + 1)), or of all 16 (one tile, column i = float i:
// the lane forms the real or the imaginary part of channel i / 2).
template <int N1, int N2, bool ONE_ROWB>
__global__ void __launch_bounds__(64 * kCellsF) onepair_mfma_fwd_kernel(const OnePairMfmaArgs a) {
  using Sh = PairShape<N1, N2>;
  constexpr int T = Sh::T, W = Sh::W;
  constexpr int XROW = N1 * 8, YROW = N2 * 8;  // bytes of a row of the operands in LDS
  extern __shared__ float4 smem4[];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int cw = wave / W, ww = wave % W;  // the wave's cell within the block, its piece of the cell's channels
  const int lane = threadIdx.x & 63, i = lane & 31, h = lane >> 5;
  const int l1 = a.l1, l2 = a.l2, lmin = a.lmin, lt = a.lt, nl = a.nl;
  const int r1 = 2 * l1 + 1, r2 = 2 * l2 + 1;
  float *ctab = reinterpret_cast<float *>(smem4);
  const int tab4 = a.nsteps_fwd * (2 * kColsF / 4);  // float4s of the table
  // per cell: x with one row of zeros behind it, y with one row of zeros on either side (the second m1 of an odd count
  // reads one row too far; its coefficient is zero, so the row must only be finite)
  const int cell4 = ((r1 + 1) * N1 + (r2 + 2) * N2) / 2;  // float4s
  float2 *xs = reinterpret_cast<float2 *>(smem4 + tab4 + cw * cell4);
  float2 *ys = xs + (r1 + 1) * N1 + N2;  // row 0 of y; the zero row sits in front of it
  {
    const float4 *src = reinterpret_cast<const float4 *>(a.coef_fwd);
    for (int e = threadIdx.x; e < tab4; e += 64 * kCellsF) smem4[e] = src[e];
  }
  long long cell = (long long)blockIdx.x * (kCellsF / W) + cw;
  const bool live = cell < a.ncells;  // a wave beyond the last cell repeats it and stores nothing
  cell = live ? cell : a.ncells - 1;
  for (int e = ww * 64 + lane; e < r1 * N1; e += 64 * W) xs[e] = a.x.ptr[cell * a.x.sb + (long long)(e / N1) * a.x.sm + (e % N1)];
  for (int e = ww * 64 + lane; e < r2 * N2; e += 64 * W) ys[e] = a.y.ptr[cell * a.y.sb + (long long)(e / N2) * a.y.sm + (e % N2)];
  if (ww == 0) {
    if (lane < N1) xs[r1 * N1 + lane] = make_float2(0.f, 0.f);
    if (lane < N2) {
      ys[lane - N2] = make_float2(0.f, 0.f);
      ys[r2 * N2 + lane] = make_float2(0.f, 0.f);
    }
  }
  // Register v of a tile belongs to part l = lmin + 8 (v / 4) + 4 h + v % 4.  cur[v]: the lane's 4 T bytes of row m of
  // that part for the m at hand (the rows of a part start at m = -l; before that the address is not used), advanced by
  // the row length after every m.  Bit v of `there`: the part exists and the wave has a cell.
  const long long rowb = a.rowb;
  unsigned long long cur[16];
  unsigned rowbv[ONE_ROWB ? 1 : 16];
  unsigned there = 0;
  static_for<16>([&](auto vc) __attribute__((always_inline)) {
    constexpr int v = decltype(vc)::value;
    cur[v] = 0;
    if constexpr (!ONE_ROWB) rowbv[v] = 0;
    static_for<2>([&](auto hc) __attribute__((always_inline)) {
      constexpr int dl = 8 * (v / 4) + 4 * decltype(hc)::value + (v % 4);
      if constexpr (dl < kNLm) {
        if (hc.value == h && dl < nl && live && a.g[dl].ptr != nullptr) {
          const FastPart P = a.g[dl];
          const long long rb = ONE_ROWB ? rowb : (long long)P.sm * 8;
          cur[v] = (unsigned long long)(P.ptr + cell * P.sb + (a.offs[dl] + a.offs_add)) +
                   (unsigned long long)((long long)(lmin + dl - lt) * rb) + (unsigned)ww * 512u + (unsigned)i * (4u * T);
          if constexpr (!ONE_ROWB) rowbv[v] = (unsigned)rb;
          there |= 1u << v;
        }
      }
    });
  });
  const int lbase = lmin + 4 * h;  // l of register v: lbase + 8 (v / 4) + v % 4
  // the lane's channel(s): (a, j), and for a wave of 64 channels (a, j + 1) as well
  const int chan = T == 4 ? ww * 64 + 2 * i : i >> 1;
  const char *xmine = reinterpret_cast<const char *>(xs + chan / N2);  // row r: + r * XROW bytes
  const char *ymine = reinterpret_cast<const char *>(ys + chan % N2);  // row r: + r * YROW
  const bool imag = (i & 1) != 0;  // one tile: the lane's float is the imaginary part
  // the lane's coefficient of step s: 192 s bytes on; the columns beyond the table's read its last one, which is zero
  const char *cmine = reinterpret_cast<const char *>(ctab + h * kColsF + (i < kColsF ? i : kColsF - 1));
  __syncthreads();

  const bool accumulate = a.accumulate != 0;
  f16v D[T];
  int at = 0;  // first step of the m at hand in the table
  for (int m = -lt; m <= lt; m++) {
    const int lo = (m - l2 > -l1) ? m - l2 : -l1, hi = (m + l2 < l1) ? m + l2 : l1;
    const int nst = (hi - lo + 2) >> 1;
    // step k: m1 = lo + 2 k + h, m2 = m - m1: the addresses of a step are those of step 0 plus constants (y runs
    // backwards: its base is the row of the last unrolled step, so that the constants are not negative)
    const char *xm = xmine + (lo + h + l1) * XROW;
    const char *ym = ymine + (m - lo - h + l2 - 2 * (kStepsM - 1)) * YROW;
    const char *cm = cmine + at * (2 * kColsF * 4);
    static_for<kStepsM>([&](auto kc) __attribute__((always_inline)) {
      constexpr int k = decltype(kc)::value;
      if (k < nst) {  // uniform
        const float2 xv = *reinterpret_cast<const float2 *>(xm + k * 2 * XROW);
        const float c = *reinterpret_cast<const float *>(cm + k * (2 * kColsF * 4));
        float p[T];
        if constexpr (T == 4) {
          const float4 yv = *reinterpret_cast<const float4 *>(ym + (kStepsM - 1 - k) * 2 * YROW);
          p[0] = fmaf(-xv.y, yv.y, xv.x * yv.x), p[1] = fmaf(xv.y, yv.x, xv.x * yv.y);
          p[2] = fmaf(-xv.y, yv.w, xv.x * yv.z), p[3] = fmaf(xv.y, yv.z, xv.x * yv.w);
        } else {
          const float2 yv = *reinterpret_cast<const float2 *>(ym + (kStepsM - 1 - k) * 2 * YROW);
          p[0] = imag ? fmaf(xv.y, yv.x, xv.x * yv.y) : fmaf(-xv.y, yv.y, xv.x * yv.x);
        }
        if constexpr (k == 0) {  // the first step of an m starts from zero (a constant operand, no registers to clear)
          f16v zero;
#pragma unroll
          for (int v = 0; v < 16; v++) zero[v] = 0.f;
#pragma unroll
          for (int e = 0; e < T; e++) D[e] = __builtin_amdgcn_mfma_f32_32x32x2f32(c, p[e], zero, 0, 0, 0);
        } else {
#pragma unroll
          for (int e = 0; e < T; e++) D[e] = __builtin_amdgcn_mfma_f32_32x32x2f32(c, p[e], D[e], 0, 0, 0);
        }
      }
    });
    // register v of the tiles: the lane's floats of row m of its part
    const int mabs = m < 0 ? -m : m;
#pragma unroll
    for (int v = 0; v < 16; v++) {
      if (((there >> v) & 1u) && lbase + (8 * (v / 4) + v % 4) >= mabs) {
        if constexpr (T == 4) {
          GlobalOut4 q = (GlobalOut4)cur[v];
          v4f o;
          o.x = D[0][v], o.y = D[1][v], o.z = D[2][v], o.w = D[3][v];
          if (accumulate) o += *q;
          *q = o;
        } else {
          GlobalOut1 q = (GlobalOut1)cur[v];
          float o = D[0][v];
          if (accumulate) o += *q;
          *q = o;
        }
      }
      cur[v] += ONE_ROWB ? (unsigned long long)rowb : (unsigned long long)rowbv[v];
    }
    at += nst;
  }
}

// ---- host side ---------------------------------------------------------------------------------------------------

struct Tables {
  float *coef;
  int nsteps;
  float *coef_fwd;
  int nsteps_fwd;
};
std::mutex g_mutex;
std::map<std::vector<int>, Tables> g_tables;  // (device, l1, l2, lmin, lt, nl, present...) -> device tables
int g_enable = 1, g_enable_fwd = 1, g_paired = 1;

int device_tables(int l1, int l2, int lmin, int lt, int nl, const std::vector<int> &present, bool paired, Tables *out) {
  int dev = 0;
  GELIB_HIP_TRY(hipGetDevice(&dev));
  std::vector<int> key = {dev, l1, l2, lmin, lt, nl, paired ? 1 : 0};
  key.insert(key.end(), present.begin(), present.end());
  std::lock_guard<std::mutex> lock(g_mutex);
  auto it = g_tables.find(key);
  if (it == g_tables.end()) {
    std::vector<std::vector<float>> C(nl);
    for (int dl = 0; dl < nl; dl++)
      if (present[dl]) {
        C[dl].resize((size_t)(2 * l1 + 1) * (2 * l2 + 1));
        cg_matrix_host(l1, l2, lmin + dl, C[dl].data());
      }
    std::vector<float> coef;
    int step = 0;
    std::vector<int> order;  // the row numbers in the order the backward kernel takes them
    if (paired) {
      for (int m = -lt; m < 0; m++) order.push_back(m), order.push_back(m + 2 * l1 + 1);
      order.push_back(0);
    } else {
      for (int m = -lt; m <= lt; m++) order.push_back(m);
    }
    for (int m : order) {
      const int dl0 = std::max(std::abs(m), lmin) - lmin;   // the first l with a row m
      const int nks = (nl - dl0 + 1) / 2;
      for (int ks = 0; ks < nks; ks++, step++) {
        for (int lane = 0; lane < 64; lane++) {
          const int col = lane & 31, h = lane >> 5;
          const int dl = dl0 + 2 * ks + h, m1 = col - l1, m2 = m - m1;
          float c = 0.f;
          if (dl < nl && present[dl] && col <= 2 * l1 && m2 >= -l2 && m2 <= l2)
            c = C[dl][(size_t)(m1 + l1) * (2 * l2 + 1) + (m2 + l2)];
          coef.push_back(c);
        }
      }
    }
    while (step % kQueue != 0) {  // idle steps: the harmless row against coefficients that are zero
      coef.insert(coef.end(), 64, 0.f);
      step++;
    }
    coef.insert(coef.end(), (size_t)kQueue * 64, 0.f);  // the queue runs kQueue steps ahead, also at the end; the start
                                                          // of the table doubles as the harmless row (512 bytes at least)
    // forward: steps over m1 (two per step), 24 columns (l) per m1: [step][h][column]
    std::vector<float> cfwd;
    int fstep = 0;
    for (int m = -lt; m <= lt; m++) {
      const int lo = std::max(-l1, m - l2), hi = std::min(l1, m + l2);
      const int nks = (hi - lo + 2) / 2;
      for (int ks = 0; ks < nks; ks++, fstep++)
        for (int h = 0; h < 2; h++)
          for (int dl = 0; dl < kColsF; dl++) {
            const int m1 = lo + 2 * ks + h, m2 = m - m1;
            float c = 0.f;
            if (dl < nl && present[dl] && m1 <= hi && std::abs(m) <= lmin + dl)
              c = C[dl][(size_t)(m1 + l1) * (2 * l2 + 1) + (m2 + l2)];
            cfwd.push_back(c);
          }
    }
    // both tables in one allocation (the forward one behind the backward one, 256-byte aligned), freed again when a
    // copy fails
    Tables t{nullptr, step, nullptr, fstep};
    const size_t bwd_bytes = (coef.size() * sizeof(float) + 255) & ~(size_t)255;
    char *d = nullptr;
    GELIB_HIP_TRY(hipMalloc((void **)&d, bwd_bytes + cfwd.size() * sizeof(float)));
    hipError_t e = hipMemcpy(d, coef.data(), coef.size() * sizeof(float), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(d + bwd_bytes, cfwd.data(), cfwd.size() * sizeof(float), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
      (void)hipFree(d);
      return record_hip_error(e, "hipMemcpy(single-pair coefficient tables)");
    }
    t.coef = (float *)d;
    t.coef_fwd = (float *)(d + bwd_bytes);
    it = g_tables.emplace(key, t).first;
  }
  *out = it->second;
  return GELIB_HIP_OK;
}

// The channel counts the backward kernel is built for.
#define GELIB_ONEPAIR_SHAPES(X) X(8, 8) X(4, 4) X(8, 16) X(16, 16) X(16, 8) X(4, 16) X(8, 2)
bool bwd_shape_built(int n1, int n2) {
#define GELIB_X(A, B) if (n1 == A && n2 == B) return true;
  GELIB_ONEPAIR_SHAPES(GELIB_X)
#undef GELIB_X
  return false;
}
void launch_bwd_shape(int n1, int n2, const OnePairMfmaArgs &a, hipStream_t s) {
#define GELIB_X(A, B)                                                                                                   \
  if (n1 == A && n2 == B)                                                                                               \
    hipLaunchKernelGGL((onepair_mfma_bwd_kernel<A, B>), dim3((unsigned)a.ncells), dim3(64 * PairShape<A, B>::W), 0, s, a);
  GELIB_ONEPAIR_SHAPES(GELIB_X)
#undef GELIB_X
}

template <int N1, int N2, bool ONE_ROWB>
int launch_fwd_one(const OnePairMfmaArgs &a, unsigned nblocks, size_t lds, hipStream_t s) {
  static std::mutex attr_mutex;
  static std::map<int, bool> attr_set;  // device -> the kernel may use 80 KB of LDS
  int dev = 0;
  GELIB_HIP_TRY(hipGetDevice(&dev));
  {
    std::lock_guard<std::mutex> lock(attr_mutex);
    if (!attr_set[dev]) {
      GELIB_HIP_TRY(hipFuncSetAttribute((const void *)onepair_mfma_fwd_kernel<N1, N2, ONE_ROWB>,
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)(80 * 1024)));
      attr_set[dev] = true;
    }
  }
  hipLaunchKernelGGL((onepair_mfma_fwd_kernel<N1, N2, ONE_ROWB>), dim3(nblocks), dim3(64 * kCellsF), lds, s, a);
  return GELIB_HIP_OK;
}
int launch_fwd_shape(int n1, int n2, bool one_rowb, const OnePairMfmaArgs &a, unsigned nblocks, size_t lds, hipStream_t s) {
#define GELIB_X(A, B)                                                                     \
  if (n1 == A && n2 == B)                                                                 \
    return one_rowb ? launch_fwd_one<A, B, true>(a, nblocks, lds, s) : launch_fwd_one<A, B, false>(a, nblocks, lds, s);
  GELIB_ONEPAIR_SHAPES(GELIB_X)
#undef GELIB_X
  return GELIB_HIP_ERR_ARG;
}

}  // namespace

// Both gradients of a non-Diag product of one x part with one y part, l1, l2 <= 15, for the channel counts listed in
// GELIB_ONEPAIR_SHAPES.  *used = 1 if the launch was made; anything else is left to the other kernels.
int onepair_mfma_vec_bwd(const VecPlan &plan, const std::vector<const gelib_part_desc *> &g,
                         const std::vector<const gelib_part_desc *> &x, const std::vector<const gelib_part_desc *> &y,
                         const std::vector<const gelib_part_desc *> &xg, const std::vector<const gelib_part_desc *> &yg,
                         bool accumulate, hipStream_t s, int *used) {
  *used = 0;
  if (!g_enable || plan.diag || x.size() != 1 || y.size() != 1 || xg.size() != 1 || yg.size() != 1 || plan.triples.empty())
    return GELIB_HIP_OK;
  std::vector<FastPart> fx, fy, fg, fxg, fyg;
  std::vector<std::pair<int, int>> lx, ly, lg;
  if (!lists_to_fast(x, plan.E, false, &fx, &lx) || !lists_to_fast(y, plan.E, false, &fy, &ly) ||
      !lists_to_fast(g, plan.E, false, &fg, &lg) || !lists_to_fast(xg, plan.E, true, &fxg, nullptr) ||
      !lists_to_fast(yg, plan.E, true, &fyg, nullptr))
    return GELIB_HIP_OK;
  const int l1 = lx[0].first, l2 = ly[0].first, n1 = lx[0].second, n2 = ly[0].second;
  if (!bwd_shape_built(n1, n2) || l1 > kMaxLm || l2 > kMaxLm) return GELIB_HIP_OK;
  const int lmin = std::abs(l1 - l2);
  int lmax = -1;
  for (auto &t : plan.triples) lmax = std::max(lmax, t.l);
  const int nl = lmax - lmin + 1;
  if (nl > kNLm || nl < 4) return GELIB_HIP_OK;  // a few values of l: the other kernels do as well
  OnePairMfmaArgs a;
  std::memset(&a, 0, sizeof(a));
  a.x = fx[0];
  a.y = fy[0];
  a.xg = fxg[0];
  a.yg = fyg[0];
  std::vector<int> present(nl, 0);
  for (auto &t : plan.triples) {
    const int dl = t.l - lmin;
    a.g[dl] = fg[t.ri];
    a.offs[dl] = t.offs;
    present[dl] = 1;
    // 64 channels per wave: the lane's 16 bytes of a row must be 16-byte aligned (block offset, row and cell strides
    // even); with 16 channels a lane loads single floats
    if (n1 * n2 >= 64 && (((t.offs) & 1) || (fg[t.ri].sm & 1) || (fg[t.ri].sb & 1) || ((uintptr_t)fg[t.ri].ptr & 15)))
      return GELIB_HIP_OK;
    if ((long long)fg[t.ri].sm * 8 * (2 * t.l + 1) >= (1LL << 32)) return GELIB_HIP_OK;  // row offsets are 32 bits
  }
  const long long ncells = plan.E[0] * plan.E[1] * plan.E[2];
  if (ncells > 0x7fffffffLL) return GELIB_HIP_OK;
  Tables t;
  const int lt = std::min(l1 + l2, lmax);
  const bool paired = g_paired && l1 == l2 && lt == 2 * l1;
  int rc = device_tables(l1, l2, lmin, lt, nl, present, paired, &t);
  if (rc) return rc;
  a.paired = paired ? 1 : 0;
  a.coef = t.coef;
  a.nsteps = t.nsteps;
  a.ncells = ncells;
  a.l1 = l1;
  a.l2 = l2;
  a.lmin = lmin;
  a.lt = lt;
  a.nl = nl;
  a.accumulate = accumulate ? 1 : 0;
  launch_bwd_shape(n1, n2, a, s);
  GELIB_HIP_TRY(hipGetLastError());
  *used = 1;
  return GELIB_HIP_OK;
}

// The product itself for the same shapes (non-Diag, l1, l2 <= 15, 4 to 22 values of l).
int onepair_mfma_vec_fwd(const VecPlan &plan, const std::vector<const gelib_part_desc *> &r,
                         const std::vector<const gelib_part_desc *> &x, const std::vector<const gelib_part_desc *> &y,
                         bool accumulate, hipStream_t s, int *used) {
  *used = 0;
  if (!g_enable_fwd || plan.diag || x.size() != 1 || y.size() != 1 || plan.triples.empty()) return GELIB_HIP_OK;
  std::vector<FastPart> fx, fy, fr;
  std::vector<std::pair<int, int>> lx, ly, lr;
  if (!lists_to_fast(x, plan.E, false, &fx, &lx) || !lists_to_fast(y, plan.E, false, &fy, &ly) ||
      !lists_to_fast(r, plan.E, true, &fr, &lr))
    return GELIB_HIP_OK;
  const int l1 = lx[0].first, l2 = ly[0].first, n1 = lx[0].second, n2 = ly[0].second;
  if (!bwd_shape_built(n1, n2) || l1 > kMaxLm || l2 > kMaxLm) return GELIB_HIP_OK;
  const int lmin = std::abs(l1 - l2);
  int lmax = -1;
  for (auto &t : plan.triples) lmax = std::max(lmax, t.l);
  const int nl = lmax - lmin + 1;
  if (nl > kNLm || nl < 4) return GELIB_HIP_OK;
  static_assert(kNLm <= kColsF, "the forward table keeps one column per value of l");
  OnePairMfmaArgs a;
  std::memset(&a, 0, sizeof(a));
  a.x = fx[0];
  a.y = fy[0];
  std::vector<int> present(nl, 0);
  bool one_rowb = true;
  for (auto &t : plan.triples) {
    const int dl = t.l - lmin;
    a.g[dl] = fr[t.ri];
    a.offs[dl] = t.offs;
    present[dl] = 1;
    // 64 channels per wave: a lane stores 16 bytes at a time (block offset, row and cell strides even, base aligned);
    // with 16 channels it stores single floats
    if (n1 * n2 >= 64 && (((t.offs) & 1) || (fr[t.ri].sm & 1) || (fr[t.ri].sb & 1) || ((uintptr_t)fr[t.ri].ptr & 15)))
      return GELIB_HIP_OK;
    if ((long long)fr[t.ri].sm * 8 >= (1LL << 32)) return GELIB_HIP_OK;  // row lengths are 32 bits
    if (a.rowb == 0) a.rowb = (long long)fr[t.ri].sm * 8;
    if (a.rowb != (long long)fr[t.ri].sm * 8) one_rowb = false;
  }
  const long long ncells = plan.E[0] * plan.E[1] * plan.E[2];
  if (ncells > 0x7fffffffLL) return GELIB_HIP_OK;
  Tables t;
  const int lt = std::min(l1 + l2, lmax);
  int rc = device_tables(l1, l2, lmin, lt, nl, present, false, &t);
  if (rc) return rc;
  a.coef_fwd = t.coef_fwd;
  a.nsteps_fwd = t.nsteps_fwd;
  a.ncells = ncells;
  a.l1 = l1;
  a.l2 = l2;
  a.lmin = lmin;
  a.lt = lt;
  a.nl = nl;
  a.accumulate = accumulate ? 1 : 0;
  // LDS of a block: the table and its cells' operands (with their rows of zeros); two blocks per compute unit fit
  // up to 80 KB each, beyond that the any-l kernels take the pair
  const int cells_per_block = n1 * n2 >= 64 ? kCellsF * 64 / (n1 * n2) : kCellsF;
  const size_t lds = (size_t)t.nsteps_fwd * 2 * kColsF * 4 +
                     (size_t)cells_per_block * ((size_t)(2 * l1 + 2) * n1 + (size_t)(2 * l2 + 3) * n2) * 8;
  if (lds > 80 * 1024) return GELIB_HIP_OK;
  rc = launch_fwd_shape(n1, n2, one_rowb, a, (unsigned)((ncells + cells_per_block - 1) / cells_per_block), lds, s);
  if (rc) return rc;
  GELIB_HIP_TRY(hipGetLastError());
  *used = 1;
  return GELIB_HIP_OK;
}

int onepair_mfma_set_option(const char *name, int value) {
  if (!std::strcmp(name, "onepair_mfma_fwd")) {
    g_enable_fwd = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "onepair_mfma_paired")) {
    g_paired = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "onepair_mfma")) {
    g_enable = value;
    return GELIB_HIP_OK;
  }
  return GELIB_HIP_ERR_ARG;
}

}  // namespace gelib_hip
