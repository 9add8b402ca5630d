// Shared host/device declarations of libgelib_hip.so (internal; the public interface is include/gelib_hip.h).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

#include "gelib_hip.h"

namespace gelib_hip {

constexpr int kMaxL = GELIB_HIP_MAX_L;
constexpr int kMaxParts = GELIB_HIP_MAX_PARTS;
constexpr int kMaxOutParts = GELIB_HIP_MAX_OUT_PARTS;
constexpr int kWave = 64;

// A part as the shape-agnostic kernels see it: 5-D strides in complex elements (0 = broadcast).
struct PartDev {
  float2 *ptr;
  long long sb, sg0, sg1, sm, sc;
};

// One part-level operation after validation and broadcasting (host side).
struct PartOp {
  PartDev r, x, y;           // r = product or its gradient
  long long E[3];            // common extents (batch, grid0, grid1)
  long long Dr[3], Dx[3], Dy[3];  // own extents of each tensor (E[d] or 1)
  int l1, l2, l, n1, n2, nout;
  int offs;
  bool diag;
};

enum PathId { kPathNone = 0, kPathGeneric = 1, kPathUnrolled = 2, kPathStaged = 3, kPathDiag6 = 4, kPathOnePair = 5, kPathLinear = 6 };

// ---- coefficient bank (cg_bank.cpp) ----
double cg_coeff(int l1, int l2, int l, int m1, int m2);
void cg_matrix_host(int l1, int l2, int l, float *out);
// Device copy of one (2l1+1)x(2l2+1) table on the current device; cached for the life of the process.
int cg_matrix_device(int l1, int l2, int l, const float **dptr);

// ---- error plumbing ----
int record_hip_error(hipError_t e, const char *what);
#define GELIB_HIP_TRY(expr)                                   \
  do {                                                        \
    hipError_t _e = (expr);                                   \
    if (_e != hipSuccess) return record_hip_error(_e, #expr); \
  } while (0)

// ---- shape-agnostic kernels (cg_generic.hip) ----
int launch_generic_fwd(const PartOp &op, bool accumulate, hipStream_t s);
int launch_generic_back0(const PartOp &op, bool accumulate, hipStream_t s);  // destination = op.x
int launch_generic_back1(const PartOp &op, bool accumulate, hipStream_t s);  // destination = op.y
int launch_zero_fill(const PartDev &d, const long long D[3], int M, int n, hipStream_t s);

// ---- scratch memory that belongs to the library (cabi.cpp): one buffer per (kind, device, stream), allocated on first
// use, grown when more is asked for, kept until the process ends.  The caller holds stream_scratch_mutex(kind) from
// the call until the last kernel that uses the buffer is on the stream (kernels of one stream run in order, so the
// next user of the buffer comes after them).  kind 0: per-cell gradients of a broadcast destination; 1: partial sums of
// backward launches that deal the pairs of a cell to several blocks.  Memory that the caller has lent for the stream
// (gelib_hip_set_stream_workspace) is used first, half of it per kind.  *out = nullptr (status OK) when the stream is
// being recorded into a graph and nothing is lent: the caller then takes its scratch-free route.
int stream_scratch(int kind, hipStream_t s, size_t bytes, void **out);
std::mutex &stream_scratch_mutex(int kind);

// ---- sums over broadcast dimensions of a gradient destination (bcast_reduce.hip) ----
// tmp: per-cell gradients packed (E0, E1, E2, rows, n); d: the destination, whose own extents D are E[k] or 1
size_t bcast_partial_bytes(const long long E[3], const long long D[3], int rows, int n);
int launch_bcast_reduce(const float2 *tmp, float2 *partial, const PartDev &d, const long long E[3], const long long D[3],
                        int rows, int n, bool accumulate, hipStream_t s);
int launch_add_into(float2 *dst, const float2 *src, long long n, bool accumulate, hipStream_t s);   // dst[i] (+)= src[i]

// ---- spherical harmonics (spharm.hip): xs = strides of x in floats over (batch, grid0, grid1, xyz, channel) ----
int launch_spharm(const PartDev &r, const float *x, const long long xs[5], const long long D[3], int L, int n,
                  bool accumulate, hipStream_t s);

// ---- sum of slices along one leading dimension (gather.hip): r[.., t, ..] (+)= sum_{k in row t} x[.., sources[k], ..] ----
int launch_gather(float2 *r, const float2 *x, const long long rs[5], const long long xs[5], const long long D[5], int dim,
                  const int *row_ptr, const int *sources, bool accumulate, hipStream_t s);

// ---- channel mixing on the matrix cores (mix.hip): r[row, :] = x[row, :] V, V = W (n_in, n_out) or W^H for W (n_out, n_in);
// strides in complex elements.  Returns 0, 10 (a HIP call failed), 11 (n_in odd or rows of x not 16-byte aligned) or 13
// (workspace missing, misaligned or smaller than mix_workspace_bytes).  The library allocates nothing here: the re-packed
// matrix goes into the caller's workspace.
size_t mix_workspace_bytes(int n_in, int n_out);
int launch_mix(float2 *r, const float2 *x, const float2 *w, long long rows, int n_in, int n_out, long long xs,
               long long rs, bool adjoint, float *ws, size_t ws_bytes, hipStream_t s);
// the same with the packed matrix in an array of the library's own device image (no workspace, nothing allocated);
// 14 when n_in and n_out need more than mix_static_scratch_bytes()
size_t mix_static_scratch_bytes();
int launch_mix_static(float2 *r, const float2 *x, const float2 *w, long long rows, int n_in, int n_out, long long xs,
                      long long rs, bool adjoint, hipStream_t s);
// wg (n_in, n_out) = sum over the rows of conj(x[row, :])^T g[row, :]; the workspace holds the partial sums
size_t mix_wgrad_workspace_bytes(long long rows, int n_in, int n_out);
int launch_mix_wgrad(float2 *wg, const float2 *x, const float2 *g, long long rows, int n_in, int n_out, long long xs,
                     long long gs, float *ws, size_t ws_bytes, hipStream_t s);
int mix_set_option(const char *name, int value);   // "mix_long": 0 keeps long rows off the LDS-staged kernel

}  // namespace gelib_hip
