// Dispatch of the unrolled backward kernels; the instantiations live in cg_unrolled_bwd_{cg,diag}{4,8}[_pad].hip so
// that they compile in parallel.
#include "cg_unrolled_dev.h"

namespace gelib_hip {

int launch_unrolled_bwd_cg4(const BwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_unrolled_bwd_cg8(const BwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_unrolled_bwd_diag4(const BwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_unrolled_bwd_diag8(const BwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_unrolled_bwd_cg4_pad(const BwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_unrolled_bwd_cg8_pad(const BwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_unrolled_bwd_diag4_pad(const BwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_unrolled_bwd_diag8_pad(const BwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_unrolled_bwd_cg6_l6(const BwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_unrolled_bwd_cg6_l6_pad(const BwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_unrolled_bwd_cg6_hi(const BwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_unrolled_bwd_cg6_hi_pad(const BwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_unrolled_bwd_one(const BwdArgs &a, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_one_triple_bwd_k1_small(const BwdArgs &a, int l1, int l2, int l, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_one_triple_bwd_k1_large(const BwdArgs &a, int l1, int l2, int l, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_one_triple_bwd_k2_small(const BwdArgs &a, int l1, int l2, int l, int nblocks, size_t lds_bytes, hipStream_t s);
int launch_one_triple_bwd_k2_large(const BwdArgs &a, int l1, int l2, int l, int nblocks, size_t lds_bytes, hipStream_t s);

// The kernel built for one triple with 16 k channels in the second operand (k = 1, 2) and at least 16 in the first.
size_t one_triple_bwd_lds_bytes(int xsize, int ysize) {   // per wave: the operands of a cell and its two gradients
  return sizeof(float2) * (size_t)(kBlock / kWave) * 2 * ((size_t)xsize + ysize);
}
// small: the triple's code fits four waves per SIMD (same rule as one_triple_small in cg_one_triple_bwd_impl.h)
int launch_one_triple_bwd(const BwdArgs &a, int k, int l1, int l2, int l, int nblocks, size_t lds_bytes, hipStream_t s) {
  if (nblocks <= 0) return GELIB_HIP_OK;
  const bool small = k * (4 * (2 * l2 + 1) + 2 * (2 * l + 1)) + 5 * (2 * l1 + 1) <= 120;
  if (k == 1) return small ? launch_one_triple_bwd_k1_small(a, l1, l2, l, nblocks, lds_bytes, s) : launch_one_triple_bwd_k1_large(a, l1, l2, l, nblocks, lds_bytes, s);
  if (k == 2) return small ? launch_one_triple_bwd_k2_small(a, l1, l2, l, nblocks, lds_bytes, s) : launch_one_triple_bwd_k2_large(a, l1, l2, l, nblocks, lds_bytes, s);
  return GELIB_HIP_ERR_ARG;
}

size_t unrolled_bwd_lds_bytes(int bank_len, int xsize, int ysize, int cells_per_block) {
  const int waves = kBlock / kWave;
  (void)bank_len;  // the coefficient bank is read with scalar loads, not staged
  return sizeof(float2) * (size_t)(1 + waves) * cells_per_block * ((size_t)xsize + ysize);
}

// Operands up to l = 4: every product (l up to 8), Diag or not, any channel counts.  Operands up to l = 6: CGproduct
// capped at l = 6 (two instantiations, power-of-two channel counts and others, five minutes of compile time each; a
// kernel for the uncapped product, l up to 12, is not built).
// ... and the part above l = 6 of such a product on its own: llo = the smallest l present.
bool unrolled_bwd_takes(bool diag, bool padded, int lcap, int lop, int llo) {
  if (lop <= kLT) return lcap <= 2 * kLT;
  if (lop > kLTMax || diag) return false;
  (void)padded;
  return lcap <= kLTMax || (llo > kLTMax && lcap <= 2 * kLTMax);
}

int unrolled_bwd_cap(int lcap, int lop, int llo) {
  if (lop > kLTMax || lcap > 2 * kLTMax) return -1;
  if (lop > kLT) return lcap <= kLTMax ? kLTMax : (llo > kLTMax ? 2 * kLTMax : -1);
  return lcap <= kLT ? kLT : 2 * kLT;
}

// smallest l the kernel that launch_unrolled_bwd picks has code for
int unrolled_bwd_lo(int lcap, int lop, int llo) { return (lop > kLT && lcap > kLTMax && llo > kLTMax) ? kLTMax + 1 : 0; }

// lcap: largest l present in the gradient; code for l above 4 is left out when the product is capped there
int launch_unrolled_bwd(const BwdArgs &a, bool diag, int lcap, int lop, int nblocks, size_t lds_bytes, hipStream_t s) {
  if (nblocks <= 0) return GELIB_HIP_OK;
  if (lop > kLT) {
    if (lcap > kLTMax)
      return a.padded ? launch_unrolled_bwd_cg6_hi_pad(a, nblocks, lds_bytes, s) : launch_unrolled_bwd_cg6_hi(a, nblocks, lds_bytes, s);
    return a.padded ? launch_unrolled_bwd_cg6_l6_pad(a, nblocks, lds_bytes, s)
                    : launch_unrolled_bwd_cg6_l6(a, nblocks, lds_bytes, s);
  }
  if (a.only_dl >= 0 && !diag && !a.padded) return launch_unrolled_bwd_one(a, nblocks, lds_bytes, s);
  if (a.padded) {
    if (diag) return lcap <= kLT ? launch_unrolled_bwd_diag4_pad(a, nblocks, lds_bytes, s)
                                 : launch_unrolled_bwd_diag8_pad(a, nblocks, lds_bytes, s);
    return lcap <= kLT ? launch_unrolled_bwd_cg4_pad(a, nblocks, lds_bytes, s)
                       : launch_unrolled_bwd_cg8_pad(a, nblocks, lds_bytes, s);
  }
  if (diag) return lcap <= kLT ? launch_unrolled_bwd_diag4(a, nblocks, lds_bytes, s)
                               : launch_unrolled_bwd_diag8(a, nblocks, lds_bytes, s);
  return lcap <= kLT ? launch_unrolled_bwd_cg4(a, nblocks, lds_bytes, s)
                     : launch_unrolled_bwd_cg8(a, nblocks, lds_bytes, s);
}

}  // namespace gelib_hip
