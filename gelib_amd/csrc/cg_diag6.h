// Argument block and table layout of the lane-per-channel Diag kernels (internal).
#pragma once

#include "cg_unrolled.h"

namespace gelib_hip {

constexpr int kL6 = 6;
constexpr int kNP = kL6 + 1;      // operand parts l = 0..6
constexpr int kNR = 2 * kL6 + 1;  // product parts l = 0..12
constexpr int kImgRows = kNP * kNP;  // rows of all operand parts together: sum of 2l+1 = 49; part l starts at row l*l
constexpr int kZeroFloats = 16384;   // zeros behind the tables: a row of zeros for up to 8192 channels
constexpr int kMaxChannels = kZeroFloats / 2;

constexpr int iabs(int a) { return a < 0 ? -a : a; }
constexpr int imin(int a, int b) { return a < b ? a : b; }
constexpr int imax(int a, int b) { return a > b ? a : b; }

// Offsets (floats) of the (2l1+1) x (2l2+1) tables of all (l1,l2,l) in the bank, and its total length.
struct TableOffsets {
  int v[kNP][kNP][kNR];
  int total;
};
constexpr TableOffsets make_table_offsets() {
  TableOffsets t{};
  int off = 0;
  for (int a = 0; a <= kL6; a++)
    for (int b = 0; b <= kL6; b++)
      for (int c = iabs(a - b); c <= a + b; c++) {
        t.v[a][b][c] = off;
        off += (2 * a + 1) * (2 * b + 1);
      }
  t.total = off;
  return t;
}
constexpr TableOffsets kTables = make_table_offsets();
constexpr int table_off(int l1, int l2, int l) { return kTables.v[l1][l2][l]; }
constexpr int kBankFloats = (kTables.total + 1) & ~1;  // even, so that the zeros behind it are 8-byte aligned

// The bank on the current device (built and uploaded on first use, kept for the life of the process): kBankFloats
// coefficients, table (l1, l2, l) at table_off(l1, l2, l), followed by kZeroFloats zeros.
int cg_table_bank(const float **out);

struct Diag6Args {
  FastPart x[kNP], y[kNP], xg[kNP], yg[kNP];  // by l; ptr == nullptr: no such part
  FastPart r[kNR];                            // product (forward) or its gradient (backward), by l
  const int *offs;    // device, [kNP][kNP][kNR]: first channel of the triple's block in part l, -1 = no such triple
  const float *bank;  // device, kBankFloats coefficients followed by kZeroFloats zeros
  long long nwaves;   // cells * groups, or cells / (64 >> lg_npad) rounded up
  long long ncells;
  int groups;         // 64-channel groups per cell (more than 32 channels)
  int lg_npad;        // log2 of the channel count rounded up to a power of two, at most 6
  int n;              // channels of every part (of every part of the wider operand when xbc or ybc is set)
  int xbc, ybc;       // CGproduct with a one-channel first / second operand: every lane reads that channel
  int offs_add;
  int accumulate;
  int want_x, want_y;  // backward: which gradients are stored (the operand of an unwanted one is never read)
  int owner[kNP];      // backward: which of the block's four waves takes the pairs with this l2
};

int launch_diag6_fwd_l6(const Diag6Args &a, hipStream_t s);  // product l up to 6
int launch_diag6_bwd_l6(const Diag6Args &a, hipStream_t s);
int launch_diag6_bwd_l6_sets(const Diag6Args &a, hipStream_t s);  // every part of y present: fixed sets of l2 per wave
// operand parts up to l = 2, product up to l = 4: a wave per cell and channel group, no barriers
int launch_diag6_small_fwd(const Diag6Args &a, hipStream_t s);
int launch_diag6_small_bwd(const Diag6Args &a, hipStream_t s);
int launch_diag6_small4_bwd(const Diag6Args &a, hipStream_t s);     // backward, operand parts up to l = 4, gradient parts up to l = 6
int launch_diag6_small4_hi_bwd(const Diag6Args &a, hipStream_t s);  // ... gradient parts l = 7, 8 only
// product parts l = 7..12 only
int launch_diag6_fwd_hi(const Diag6Args &a, hipStream_t s);
int launch_diag6_bwd_hi(const Diag6Args &a, hipStream_t s);
int launch_diag6_fwd_hi_packed(const Diag6Args &a, hipStream_t s);  // several cells per wave (lg_npad < 6)
int launch_diag6_bwd_hi_packed(const Diag6Args &a, hipStream_t s);
// operand parts up to l = 4, product up to l = 8
int launch_diag6_fwd_l8(const Diag6Args &a, hipStream_t s);
int launch_diag6_bwd_l8(const Diag6Args &a, hipStream_t s);
int launch_diag6_fwd_l8_packed(const Diag6Args &a, hipStream_t s);
int launch_diag6_bwd_l8_packed(const Diag6Args &a, hipStream_t s);
int launch_diag6_fwd_l6_packed(const Diag6Args &a, hipStream_t s);  // several cells per wave (lg_npad < 6)
int launch_diag6_bwd_l6_packed(const Diag6Args &a, hipStream_t s);

}  // namespace gelib_hip
