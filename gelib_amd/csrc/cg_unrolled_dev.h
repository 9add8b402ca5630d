// Kernel argument blocks and launch entry points of the unrolled small-l kernels (internal).
#pragma once

#include <type_traits>
#include <utility>

#include "cg_unrolled.h"

namespace gelib_hip {

constexpr int kFastIn = kLTMax + 1;       // operand parts l = 0..kLTMax
constexpr int kFastOut = 2 * kLTMax + 1;  // product parts l = 0..2*kLTMax
constexpr int kBlock = 256;

struct FwdArgs {
  FastPart x[kFastIn], y[kFastIn];  // in list order (ascending l)
  FastPart r[kFastOut];             // indexed by l itself; absent parts have ptr == nullptr
  const PairRec *pairs;  // device
  const float *bank;     // device, concatenated coefficient tables
  long long ncells;
  int npairs;
  int offs_add;     // extra channel offset (part-level calls)
  int accumulate;
  long long tile;                  // cells per tile; the blocks of one tile are consecutive
  int blocks_per_tile;
  int first_block[kMaxPairs + 1];  // inside a tile, blocks [first_block[p], first_block[p+1]) work on pair p
  int cpb[kMaxPairs];              // cells per block of pair p
};

struct BwdArgs {
  FastPart x[kFastIn], y[kFastIn], xg[kFastIn], yg[kFastIn];  // in list order (ascending l)
  FastPart g[kFastOut];                                       // indexed by l itself; absent parts have ptr == nullptr
  const PairRec *pairs;
  const float *bank;
  long long ncells;
  int npairs;
  int nx, ny;       // number of x / y parts
  int offs_add;
  int accumulate;
  int want_x, want_y;
  int bank_len;     // floats
  int padded;       // some channel count is not a power of two (lanes beyond the real channels idle)
  int zero_off;     // even offset (floats) in the bank of a run of zeros as long as the largest coefficient table
  int xsize, ysize; // complex elements of one cell's packed x / y image
  int xrows[kFastIn], yrows[kFastIn];  // 2l+1 of each x / y part
  int cells_per_block;
  int only_dl;      // -1, or: the call has one triple, l = |l1 - l2| + only_dl (the kernel built for that case)
  // Launches with few cells: the pairs of a cell are dealt to pair_split blocks (by PairRec::cost_rank), each of which
  // writes the sums of its pairs into part_x / part_y, [split][cell][packed image of the parts]; a second small kernel
  // adds the pair_split images of a cell in their order and writes the gradients.  1: one block takes all pairs.
  int pair_split;
  float2 *part_x, *part_y;
};

size_t unrolled_bwd_lds_bytes(int bank_len, int xsize, int ysize, int cells_per_block);

// Compile-time loop: f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N-1>{}).
template <int... Is, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, Is...>, F &&f) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, static_cast<F &&>(f));
}

// Kernel-argument arrays must only be indexed with compile-time constants: a run-time index (or a chain of
// selects between entries, which the optimiser folds back into one) makes the compiler keep a copy of the
// argument block in scratch memory.  These pick an entry by OR-ing together masked copies of every entry, which
// stays scalar arithmetic on values already loaded from the argument block.
template <int N>
__device__ __forceinline__ FastPart pick_part(const FastPart (&arr)[N], int i) {
  unsigned long long ptr = 0, sb = 0;
  unsigned sm = 0, n = 0;
  static_for<N>([&](auto k) __attribute__((always_inline)) {
    const unsigned long long m64 = (i == k.value) ? ~0ull : 0ull;
    const unsigned m32 = (i == k.value) ? ~0u : 0u;
    ptr |= m64 & (unsigned long long)arr[k.value].ptr;
    sb |= m64 & (unsigned long long)arr[k.value].sb;
    sm |= m32 & (unsigned)arr[k.value].sm;
    n |= m32 & (unsigned)arr[k.value].n;
  });
  FastPart r;
  r.ptr = (float2 *)ptr;
  r.sb = (long long)sb;
  r.sm = (int)sm;
  r.n = (int)n;
  return r;
}
template <int N>
__device__ __forceinline__ int pick_int(const int (&arr)[N], int i) {
  unsigned r = 0;
  static_for<N>([&](auto k) __attribute__((always_inline)) { r |= ((i == k.value) ? ~0u : 0u) & (unsigned)arr[k.value]; });
  return (int)r;
}

// ti: channels of the first operand handled per thread (1, 2 or 4); must divide every n1.
// lop: largest l of an operand (above kLT: the kernel for l up to kLTMax -- unrolled_fwd_takes says when it exists)
bool unrolled_fwd_takes(bool diag, int ti, int lcap, int lop);
int launch_unrolled_fwd(const FwdArgs &a, bool diag, int ti, int lcap, int lop, int nblocks, size_t lds_bytes, hipStream_t s);
// lcap: largest l present in the gradient; lop: largest l of an operand (above kLT: the kernel for l up to kLTMax, which
// exists for CGproduct with power-of-two channel counts and lcap <= kLTMax only -- unrolled_bwd_takes says so)
bool unrolled_bwd_takes(bool diag, bool padded, int lcap, int lop, int llo);
// largest l the backward kernel that launch_unrolled_bwd picks has code for (its step records are laid out for it),
// or -1 when no backward kernel takes the vector
int unrolled_bwd_cap(int lcap, int lop, int llo);
int unrolled_bwd_lo(int lcap, int lop, int llo);   // ... and the smallest (llo: smallest l present in the gradient)
int launch_unrolled_bwd(const BwdArgs &a, bool diag, int lcap, int lop, int nblocks, size_t lds_bytes, hipStream_t s);
// adds the pair_split partial images of every cell and writes xg / yg (nblocks = blocks of a.cells_per_block cells)
int launch_unrolled_bwd_sum_splits(const BwdArgs &a, int nblocks, hipStream_t s);
// one triple (a.only_dl >= 0), second operand of 16 k channels (k = 1, 2), first operand a power of two >= 16
size_t one_triple_bwd_lds_bytes(int xsize, int ysize);
int launch_one_triple_bwd(const BwdArgs &a, int k, int l1, int l2, int l, int nblocks, size_t lds_bytes, hipStream_t s);

}  // namespace gelib_hip
