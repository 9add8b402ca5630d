// Kernel argument blocks and launch entry points of the unrolled small-l kernels (internal).
#pragma once

#include <type_traits>
#include <utility>

#include "cg_unrolled.h"

namespace gelib_hip {

constexpr int kFastIn = kLT + 1;       // operand parts l = 0..kLT
constexpr int kFastOut = 2 * kLT + 1;  // product parts l = 0..2*kLT
constexpr int kBlock = 256;

struct FwdArgs {
  FastPart x[kFastIn], y[kFastIn], r[kFastOut];
  const PairRec *pairs;  // device
  const float *bank;     // device, concatenated coefficient tables
  long long ncells;
  int npairs;
  int offs_add;     // extra channel offset (part-level calls)
  int accumulate;
  int first_block[kMaxPairs + 1];  // blocks [first_block[p], first_block[p+1]) work on pair p
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
  int xsize, ysize; // complex elements of one cell's packed x / y image
  int xrows[kFastIn], yrows[kFastIn];  // 2l+1 of each x / y part
  int cells_per_block;
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

// Kernel-argument arrays must only be indexed with compile-time constants (a run-time index, or a loop the
// optimiser unrolls late, makes the compiler keep a copy of the whole argument block in scratch memory); these
// pick an entry with scalar selects instead.
template <int N>
__device__ __forceinline__ FastPart pick_part(const FastPart (&arr)[N], int i) {
  FastPart r = arr[0];
  static_for<N>([&](auto k) __attribute__((always_inline)) {
    if (k.value > 0 && i == k.value) r = arr[k.value];
  });
  return r;
}
template <int N>
__device__ __forceinline__ int pick_int(const int (&arr)[N], int i) {
  int r = arr[0];
  static_for<N>([&](auto k) __attribute__((always_inline)) {
    if (k.value > 0 && i == k.value) r = arr[k.value];
  });
  return r;
}

// ti: channels of the first operand handled per thread (1, 2 or 4); must divide every n1.
int launch_unrolled_fwd(const FwdArgs &a, bool diag, int ti, int nblocks, hipStream_t s);
// lcap: largest l present in the gradient
int launch_unrolled_bwd(const BwdArgs &a, bool diag, int lcap, int nblocks, size_t lds_bytes, hipStream_t s);

}  // namespace gelib_hip
