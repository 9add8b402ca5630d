// Channel mixing of a part:  r[row, o] = sum_c x[row, c] * V[c, o]  over complex64, row = (cell, m), with
// V = W (n_in, n_out) or V = W^H for W (n_out, n_in).  This is what consumes a product in the reference's Python layer:
// SO3vec.__mul__(SO3weights) is one torch.matmul(part, W) per l (python/src/gelib/SO3vec.py:174-177,
// python/src/gelib/SO3weights.py:75-85); the adjoint form is the gradient of that matmul with respect to the part.
//
// The matrix is tall and skinny (hundreds of thousands of rows, n_out of 16..64 or n_in of 16..64), which library
// complex GEMMs handle poorly.  Here the complex product is run as a real one on the matrix cores: a row of x is a real
// vector of 2 n_in floats as it lies in memory, V becomes the real (2 n_in, 2 n_out) matrix
//     [ Re V   Im V ]   (rows 2c, 2c+1; columns 2o, 2o+1)
//     [-Im V   Re V ]
// and the real product row is the complex result as it lies in memory.  v_mfma_f32_32x32x2_f32 multiplies a 32 x 2 block
// of x by a 2 x 32 block of that matrix; lane (i, h) = (lane % 32, lane / 32) supplies x[row i][k + h] and V'[k + h][col i].
// V' is re-packed once per call into exactly the order the lanes read it (pack_kernel) and stays in L2.
// Bound: HBM for n_out <= 16 (8 B of x per 8 n_out flops is 16 flop/B at n_out = 16, below the fp32 matrix-core ridge of
// 157.3 TF / 8 TB/s = 19.7 flop/B), the matrix cores above that.
//
// Kernels: mix_kernel (a lane is tied to a row; any shape), mix_long_kernel (long rows into 16 channels or fewer),
// mix_wide_kernel (16 channels or fewer into many: the gradient of a part), wgrad_kernel + wgrad_sum_kernel (the
// gradient of the matrix).  In all of them a load never sits behind a branch (an address is clamped and the value
// zeroed where it is used instead): behind a branch the compiler waits for every load in flight, not only the one
// needed, which stops the loads of the next step from overlapping the matrix instructions of this one.
//
// mix_kernel: a wave owns 32 RT rows and CTW tiles of 32 output floats, and walks the reduction 32 floats (128 B of
// every row) at a time: lane (i, h) reads the 16 floats of its row that start at 16 h.
#include <algorithm>
#include <map>
#include <mutex>
#include <string>

#include "cg_common.h"

namespace gelib_hip {

namespace {

typedef float f16v __attribute__((ext_vector_type(16)));

struct MixArgs {
  const float *x;    // rows x (2 n_in) floats, row stride xs floats
  const float *vp;   // packed V', in the order of pack_kernel
  float *r;          // rows x (2 n_out) floats, row stride rs floats
  long long rows, xs, rs;
  int k2;            // 2 n_in
  int n2;            // 2 n_out
  int nq;            // steps of the reduction: ceil(k2 / 32), or ceil(k2 / 128) for the long-step kernel
  int ct_total;      // tiles of 32 output floats, padded to a multiple of CTW
  int wide_store;    // rows of r are 16-byte aligned and n2 is a multiple of 4: results leave through LDS, 512 B a row
};

// V'[kf][col] for kf = 2 P q + P h + 4 s + e (4 s + e < P), col = 32 ct + i, stored at
// (((q * ct_total + ct) * P / 4 + s) * 64 + lane) * 4 + e: a wave reads 1 KB in one piece per load instruction.
// P = 2^lg_p floats per lane and step, 16 for the short-step kernel and 64 for the long-step one
__global__ void __launch_bounds__(256) pack_kernel(const float2 *w, float *vp, int n_in, int n_out, int nq, int ct_total,
                                                   int adjoint, int lg_p) {
  const long long total = ((long long)nq * ct_total * 64) << lg_p;
  for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long long)gridDim.x * blockDim.x) {
    const int e = (int)(idx & 3), lane = (int)((idx >> 2) & 63);
    const int sg = (int)((idx >> 8) & ((1 << (lg_p - 2)) - 1));
    const long long tile = idx >> (lg_p + 6);
    const int ct = (int)(tile % ct_total), q = (int)(tile / ct_total);
    const int kf = ((2 * q + (lane >> 5)) << lg_p) + 4 * sg + e, col = 32 * ct + (lane & 31);
    const int c = kf >> 1, o = col >> 1;
    float v = 0.f;
    if (c < n_in && o < n_out) {
      float2 e = adjoint ? w[(long long)o * n_in + c] : w[(long long)c * n_out + o];
      if (adjoint) e.y = -e.y;
      const bool im_in = kf & 1, im_out = col & 1;
      v = im_in ? (im_out ? e.x : -e.y) : (im_out ? e.y : e.x);
    }
    vp[idx] = v;
  }
}

template <int RT, int CTW>
struct Operands {
  float4 a[RT][4];
  float4 b[CTW][4];
};

template <int RT, int CTW, bool PIPE>
__global__ void __launch_bounds__(256) mix_kernel(const MixArgs p) {
  const int lane = threadIdx.x & 63, i = lane & 31, h = lane >> 5;
  const long long wave = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const long long row0 = wave * (32 * RT);
  constexpr bool kWide = !PIPE && CTW == 4;   // the variant for short reductions into many tiles (gradient of a part)
  if (row0 >= p.rows && !(kWide && p.wide_store)) return;   // with wide stores every wave reaches the barriers below
  const int ct0 = blockIdx.y * CTW;
  const float *xrow[RT];
#pragma unroll
  for (int t = 0; t < RT; t++) {
    long long row = row0 + 32 * t + i;
    if (row > p.rows - 1) row = p.rows - 1;   // rows past the end repeat the last one; their results are not stored
    xrow[t] = p.x + row * p.xs + 16 * h;
  }
  const float *vp = p.vp + (long long)ct0 * 1024 + lane * 4;
  const long long vstep = (long long)p.ct_total * 1024;

  f16v acc[RT][CTW];
#pragma unroll
  for (int t = 0; t < RT; t++)
#pragma unroll
    for (int c = 0; c < CTW; c++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[t][c][v] = 0.f;

  // k2 is a multiple of 4, so a float4 of a row is inside it or outside it as a whole; one that would start outside
  // is read from the row's end instead (no branch around a load, so loads stay in flight across the matrix
  // instructions) and replaced by zeros when it is used
  auto load = [&](int q, Operands<RT, CTW> &o) {
#pragma unroll
    for (int t = 0; t < RT; t++)
#pragma unroll
      for (int s = 0; s < 4; s++) {
        const int kf = 32 * q + 16 * h + 4 * s;
        const int at = kf < p.k2 ? 32 * q + 4 * s : p.k2 - 4 - 16 * h;
        o.a[t][s] = *(const float4 *)(xrow[t] + at);
      }
#pragma unroll
    for (int c = 0; c < CTW; c++)
#pragma unroll
      for (int s = 0; s < 4; s++) o.b[c][s] = *(const float4 *)(vp + q * vstep + c * 1024 + 256 * s);
  };
  auto compute = [&](int q, const Operands<RT, CTW> &o) {
#pragma unroll
    for (int s = 0; s < 4; s++) {
      const bool inside = 32 * q + 16 * h + 4 * s < p.k2;
#pragma unroll
      for (int e = 0; e < 4; e++)
#pragma unroll
        for (int t = 0; t < RT; t++)
#pragma unroll
          for (int c = 0; c < CTW; c++) {
            const float ar = e == 0 ? o.a[t][s].x : (e == 1 ? o.a[t][s].y : (e == 2 ? o.a[t][s].z : o.a[t][s].w));
            const float av = inside ? ar : 0.f;
            const float bv = e == 0 ? o.b[c][s].x : (e == 1 ? o.b[c][s].y : (e == 2 ? o.b[c][s].z : o.b[c][s].w));
            acc[t][c] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[t][c], 0, 0, 0);
          }
    }
  };

  if (PIPE) {
    Operands<RT, CTW> o0, o1;
    load(0, o0);
    int q = 0;
    for (; q + 2 < p.nq; q += 2) {   // no branch inside: the waits count exactly the loads issued after the ones needed
      load(q + 1, o1);
      __builtin_amdgcn_sched_barrier(0);   // keep the loads ahead of the matrix instructions of the other buffer
      compute(q, o0);
      __builtin_amdgcn_sched_barrier(0);
      load(q + 2, o0);
      __builtin_amdgcn_sched_barrier(0);
      compute(q + 1, o1);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (q + 1 < p.nq) {
      load(q + 1, o1);
      compute(q, o0);
      compute(q + 1, o1);
    } else {
      compute(q, o0);
    }
  } else {
    Operands<RT, CTW> o0;
    for (int q = 0; q < p.nq; q++) {
      load(q, o0);
      compute(q, o0);
    }
  }

  // register v of the 32 x 32 result holds row 8 (v / 4) + 4 h + (v % 4), column i
  if constexpr (kWide) {
    // Straight from the registers a store instruction covers two rows of 128 B.  Through LDS the 32 x 128 floats of a
    // row tile leave as two rows of 512 B per instruction.
    constexpr int kPitch = 128;   // four waves: 64 KB in all
    __shared__ float4 out4[4][32 * kPitch / 4];
    if (p.wide_store) {
      float *tile = (float *)out4[threadIdx.x >> 6];
#pragma unroll
      for (int t = 0; t < RT; t++) {
        if (t > 0) __syncthreads();
#pragma unroll
        for (int c = 0; c < CTW; c++)
#pragma unroll
          for (int v = 0; v < 16; v++) tile[(8 * (v / 4) + 4 * h + (v % 4)) * kPitch + 32 * c + i] = acc[t][c][v];
        __syncthreads();
        const int col = 32 * ct0 + 4 * i;
#pragma unroll
        for (int u = 0; u < 16; u++) {
          const long long row = row0 + 32 * t + 2 * u + h;
          const float4 v = *(const float4 *)(tile + (2 * u + h) * kPitch + 4 * i);
          if (row < p.rows && col < p.n2) *(float4 *)(p.r + row * p.rs + col) = v;
        }
      }
      return;
    }
  }
#pragma unroll
  for (int t = 0; t < RT; t++)
#pragma unroll
    for (int c = 0; c < CTW; c++) {
      const int col = 32 * (ct0 + c) + i;
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const long long row = row0 + 32 * t + 8 * (v / 4) + 4 * h + (v % 4);
        if (row < p.rows && col < p.n2) p.r[row * p.rs + col] = acc[t][c][v];
      }
    }
}

// Long reductions (n_in of hundreds or thousands) into one tile of output (n_out <= 16).  In the kernel above a lane
// is tied to a row, so one load instruction touches 64 different cache lines and uses 16 B of each, and a row is visited
// 128 B at a time.  Here a wave of its own (a 64-thread block) reads 32 rows 512 B at a time with loads whose lanes run
// along the row (two rows per instruction) and turns the tile through LDS into the layout of the matrix cores.  The loads
// of the next tile and of the next 64 floats per lane of V' are issued before the 64 matrix instructions of a step and
// waited for after them; the operands of x come out of LDS four matrix instructions at a time.
constexpr int kLongChunk = 128;            // floats of a row per step
constexpr int kLongPitch = kLongChunk + 4; // LDS row pitch: consecutive rows start 4 banks apart

__global__ void __launch_bounds__(64, 8) mix_long_kernel(const MixArgs p) {
  __shared__ float4 tile4[32 * kLongPitch / 4];
  float *tile = (float *)tile4;
  const int lane = threadIdx.x, i = lane & 31, h = lane >> 5;
  const long long row0 = (long long)blockIdx.x * 32;
  const float *xbase = p.x + row0 * p.xs;
  const long long left = p.rows - 1 - row0;
  const int lim = left < 31 ? (int)left : 31;   // rows past the end repeat the last one; their results are not stored
  const unsigned pitch = (unsigned)p.xs;
  const float *vp = p.vp + lane * 4;

  f16v acc;
#pragma unroll
  for (int v = 0; v < 16; v++) acc[v] = 0.f;

  float4 stage[16], b0[16], b1[16];
  // instruction u covers rows 2u and 2u+1, lane (i, h) the 16 bytes at float 4 i of row 2u + h; a chunk that starts
  // outside the row (k2 is a multiple of 4, so it is inside or outside as a whole) is read from the row's end instead
  // and replaced by zeros on its way into LDS
  auto fetch_x = [&](int q) {
    const int kf = q * kLongChunk + 4 * i;
    const unsigned col = kf < p.k2 ? kf : p.k2 - 4;
#pragma unroll
    for (int u = 0; u < 16; u++) {
      const int r = 2 * u + h < lim ? 2 * u + h : lim;
      unsigned off = (unsigned)r * pitch + col;
      asm volatile("" : "+v"(off));
      stage[u] = *(const float4 *)(xbase + off);
    }
  };
  auto fetch_v = [&](int q, float4 (&b)[16]) {
#pragma unroll
    for (int s = 0; s < 16; s++) b[s] = *(const float4 *)(vp + (long long)q * 4096 + 256 * s);
  };
  auto step = [&](int q, const float4 (&bcur)[16], float4 (&bnext)[16]) {
    __syncthreads();   // the reads of the previous tile are over
    const bool inside = q * kLongChunk + 4 * i < p.k2;
#pragma unroll
    for (int u = 0; u < 16; u++)
      *(float4 *)(tile + (2 * u + h) * kLongPitch + 4 * i) = inside ? stage[u] : make_float4(0.f, 0.f, 0.f, 0.f);
    __syncthreads();
    if (q + 1 < p.nq) {
      fetch_v(q + 1, bnext);
      fetch_x(q + 1);
    }
    const float *arow = tile + i * kLongPitch + 64 * h;
    float4 a0 = *(const float4 *)arow, a1 = *(const float4 *)(arow + 4);
#pragma unroll
    for (int s = 0; s < 16; s += 2) {
      const float4 c0 = a0, c1 = a1;
      if (s + 2 < 16) {   // the next two operands leave LDS while these eight instructions run
        a0 = *(const float4 *)(arow + 4 * (s + 2));
        a1 = *(const float4 *)(arow + 4 * (s + 3));
      }
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(c0.x, bcur[s].x, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(c0.y, bcur[s].y, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(c0.z, bcur[s].z, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(c0.w, bcur[s].w, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(c1.x, bcur[s + 1].x, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(c1.y, bcur[s + 1].y, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(c1.z, bcur[s + 1].z, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(c1.w, bcur[s + 1].w, acc, 0, 0, 0);
    }
  };
  fetch_v(0, b0);
  fetch_x(0);
  for (int q = 0; q < p.nq; q += 2) {
    step(q, b0, b1);
    if (q + 1 < p.nq) step(q + 1, b1, b0);
  }

#pragma unroll
  for (int v = 0; v < 16; v++) {
    const long long row = row0 + 8 * (v / 4) + 4 * h + (v % 4);
    if (row < p.rows && i < p.n2) p.r[row * p.rs + i] = acc[v];
  }
}

// Short reductions (n_in <= 16, one step) into many tiles of output: the gradient of a part after a layer that mixed it
// down to 16 channels.  The work is all in the stores.  A wave of its own keeps its 64 rows of x in registers and walks
// along the output 64 floats (two tiles) at a time: the next two tiles of V' are fetched while the 64 matrix
// instructions of this pair run, and the 64 x 64 results leave through LDS as four rows of 256 B per store instruction.
constexpr int kWidePitch = 64 + 4;

struct WideArgs {
  MixArgs m;
  int pairs;            // pairs of output tiles (ct_total / 2)
  int parts;            // waves per 64 rows
};

// The block is one wave and LDS serves the instructions of a wave in the order they were issued, so a write of one lane
// followed by a read of another needs no barrier instruction -- only that the compiler keeps the order.
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__global__ void __launch_bounds__(64, 8) mix_wide_kernel(const WideArgs w) {
  const MixArgs &p = w.m;
  __shared__ float4 tile4[64 * kWidePitch / 4];
  float *tile = (float *)tile4;
  const int lane = threadIdx.x, i = lane & 31, h = lane >> 5;
  const int part = blockIdx.x % w.parts;
  const long long row0 = (long long)(blockIdx.x / w.parts) * 64;
  // the waves of one group of rows take the pairs of tiles in turn (wave `part` takes pairs part, part + parts, ...):
  // they start together, so at any time they write neighbouring pieces of the same rows
  const int npairs = (w.pairs - part + w.parts - 1) / w.parts;
  if (npairs <= 0) return;   // the whole block leaves
  // the 32 floats (or fewer) of the lane's two rows of x; a float4 that would start outside the row is read from the
  // row's end instead and zeroed
  float4 a[2][4];
#pragma unroll
  for (int t = 0; t < 2; t++) {
    long long row = row0 + 32 * t + i;
    if (row > p.rows - 1) row = p.rows - 1;
    const float *xr = p.x + row * p.xs;
#pragma unroll
    for (int s = 0; s < 4; s++) {
      const int kf = 16 * h + 4 * s;
      const float4 v = *(const float4 *)(xr + (kf < p.k2 ? kf : p.k2 - 4));
      a[t][s] = kf < p.k2 ? v : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  }
  const float *vp = p.vp + lane * 4;
  float4 b0[2][4], b1[2][4];
  auto load = [&](int cp, float4 (&b)[2][4]) {
#pragma unroll
    for (int c = 0; c < 2; c++)
#pragma unroll
      for (int s = 0; s < 4; s++) b[c][s] = *(const float4 *)(vp + (long long)(2 * cp + c) * 1024 + 256 * s);
  };
  auto pair = [&](int cp, const float4 (&b)[2][4]) {
    f16v acc[2][2];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
      for (int c = 0; c < 2; c++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[t][c][v] = 0.f;
#pragma unroll
    for (int s = 0; s < 4; s++)
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int c = 0; c < 2; c++) {
          acc[t][c] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t][s].x, b[c][s].x, acc[t][c], 0, 0, 0);
          acc[t][c] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t][s].y, b[c][s].y, acc[t][c], 0, 0, 0);
          acc[t][c] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t][s].z, b[c][s].z, acc[t][c], 0, 0, 0);
          acc[t][c] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t][s].w, b[c][s].w, acc[t][c], 0, 0, 0);
        }
    wave_sync();   // the reads of the previous pair come first
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
      for (int c = 0; c < 2; c++)
#pragma unroll
        for (int v = 0; v < 16; v++)
          tile[(32 * t + 8 * (v / 4) + 4 * h + (v % 4)) * kWidePitch + 32 * c + i] = acc[t][c][v];
    wave_sync();
    const int col = 64 * cp + 4 * (lane & 15);
#pragma unroll
    for (int u = 0; u < 16; u++) {
      const int lr = 4 * u + (lane >> 4);
      const float4 v = *(const float4 *)(tile + lr * kWidePitch + 4 * (lane & 15));
      if (row0 + lr < p.rows && col < p.n2) *(float4 *)(p.r + (row0 + lr) * p.rs + col) = v;
    }
  };
  auto at = [&](int k) { return part + k * w.parts; };
  load(at(0), b0);
  int k = 0;
  for (; k + 2 < npairs; k += 2) {   // no branch inside, and fences: the next tiles stay ahead of these sums
    load(at(k + 1), b1);
    __builtin_amdgcn_sched_barrier(0);
    pair(at(k), b0);
    __builtin_amdgcn_sched_barrier(0);
    load(at(k + 2), b0);
    __builtin_amdgcn_sched_barrier(0);
    pair(at(k + 1), b1);
    __builtin_amdgcn_sched_barrier(0);
  }
  if (k + 1 < npairs) {
    load(at(k + 1), b1);
    pair(at(k), b0);
    pair(at(k + 1), b1);
  } else {
    pair(at(k), b0);
  }
}

int g_mix_long = 1;
int g_mix_wide_store = 1;
int g_mix_wide = 1;
int g_mix_wide_waves = 40960;

template <int RT, int CTW, bool PIPE>
void launch(const MixArgs &a, hipStream_t s) {
  const long long waves = (a.rows + 32 * RT - 1) / (32 * RT);
  dim3 grid((unsigned)((waves + 3) / 4), (unsigned)(a.ct_total / CTW));
  hipLaunchKernelGGL((mix_kernel<RT, CTW, PIPE>), grid, dim3(256), 0, s, a);
}

}  // namespace

// Floats of the re-packed matrix: nq steps of (2 << lg_p) floats of a row, ct_total tiles of 32 output floats.
static long long packed_floats(int n_in, int n_out, int lg_p) {
  const int k2 = 2 * n_in, tiles = (2 * n_out + 31) / 32;
  const int ctw = tiles > 2 ? 4 : tiles;
  const long long ct_total = (tiles + ctw - 1) / ctw * ctw;
  const long long nq = (k2 + (2 << lg_p) - 1) / (2 << lg_p);
  return (nq * ct_total * 64) << lg_p;
}

// Bytes of workspace launch_mix needs at most for these sizes (the long-row kernel packs in steps of 128 floats, the
// others in steps of 32; which one runs also depends on the row stride, so the larger of the two is asked for).
size_t mix_workspace_bytes(int n_in, int n_out) {
  if (n_in <= 0 || n_out <= 0) return 0;
  return sizeof(float) * (size_t)std::max(packed_floats(n_in, n_out, 4), packed_floats(n_in, n_out, 6));
}

// 0 on success, 10 when a HIP call fails, 11 when the shape is not one this kernel takes (n_in odd, strides that break
// the 16-byte alignment of a row), 13 when the workspace is missing, not 16-byte aligned or too small.  The workspace
// (device memory, mix_workspace_bytes) receives the re-packed matrix; the kernels of this call read it, so the caller
// keeps it until they have run.
int launch_mix(float2 *r, const float2 *x, const float2 *w, long long rows, int n_in, int n_out, long long xs,
               long long rs, bool adjoint, float *ws, size_t ws_bytes, hipStream_t s) {
  if (rows == 0 || n_out == 0) return 0;
  if (n_in <= 0 || (n_in & 1) || (xs & 1) || ((uintptr_t)x & 15)) return 11;
  if (rows > (1LL << 38)) return 11;
  MixArgs a;
  a.x = (const float *)x;
  a.r = (float *)r;
  a.rows = rows;
  a.xs = 2 * xs;
  a.rs = 2 * rs;
  a.k2 = 2 * n_in;
  a.n2 = 2 * n_out;
  a.wide_store = (n_out % 2 == 0 && rs % 2 == 0 && ((uintptr_t)r & 15) == 0) ? g_mix_wide_store : 0;
  const int tiles = (a.n2 + 31) / 32;
  // rows of 2 KB and more into a single tile of output: the LDS-staged kernel (32 rows must lie within 2^32 floats)
  const bool long_rows = tiles == 1 && a.k2 >= 4 * kLongChunk && a.xs < (1LL << 26) && g_mix_long;
  const bool wide = tiles > 2;
  const int ctw = wide ? 4 : tiles;
  a.ct_total = (tiles + ctw - 1) / ctw * ctw;
  const int lg_p = long_rows ? 6 : 4;
  a.nq = (a.k2 + (2 << lg_p) - 1) / (2 << lg_p);
  const long long total = ((long long)a.nq * a.ct_total * 64) << lg_p;
  if (!ws || ((uintptr_t)ws & 15) || ws_bytes < (size_t)total * sizeof(float)) return 13;
  float *vp = ws;
  a.vp = vp;
  hipLaunchKernelGGL(pack_kernel, dim3((unsigned)std::min<long long>((total + 255) / 256, 4096)), dim3(256), 0, s, w, vp,
                     n_in, n_out, a.nq, a.ct_total, adjoint ? 1 : 0, lg_p);
  if (long_rows) {
    const long long blocks = (rows + 31) / 32;
    if (blocks > 0x7fffffffLL) return 11;
    hipLaunchKernelGGL(mix_long_kernel, dim3((unsigned)blocks), dim3(64), 0, s, a);
  } else if (!wide) {
    if (ctw == 1) launch<2, 1, true>(a, s);
    else launch<2, 2, true>(a, s);
  } else if (a.nq == 1 && a.wide_store && g_mix_wide) {
    WideArgs wa;
    wa.m = a;
    wa.pairs = a.ct_total / 2;
    const long long groups = (rows + 63) / 64;
    // enough waves for some ten rounds over the chip, but no wave with fewer than four pairs of tiles
    long long parts = std::max<long long>(1, std::min<long long>(g_mix_wide_waves / groups, wa.pairs / 4));
    wa.parts = (int)parts;
    if (groups * wa.parts > 0x7fffffffLL) return 11;
    hipLaunchKernelGGL(mix_wide_kernel, dim3((unsigned)(groups * wa.parts)), dim3(64), 0, s, wa);
  } else if (a.nq <= 2) {
    launch<2, 4, false>(a, s);
  } else {
    launch<1, 4, true>(a, s);
  }
  return hipGetLastError() == hipSuccess ? 0 : 10;
}

// ---- the same product for callers that cannot allocate -------------------------------------------------------------
// Code under graph capture, tight serving loops and harnesses that forbid hipMalloc have no workspace to pass.  For them
// the packed matrix goes into an array that is part of the library's device image: every GPU the library runs on holds
// its own copy (kStaticScratchBytes, until the process ends) at its own address.  In host code the array's name is only a
// stand-in for that address, so it is never passed to a kernel or a copy: the address is asked for once per device with
// hipGetSymbolAddress, with that device current, and from then on only that pointer is used.  Every call on a GPU
// shares that GPU's array: calls that overlap on one GPU (two streams, two host threads) race on it.  Nothing in it has
// to start at zero, since the pack kernel writes every float of the region a call reads, padding included.
constexpr size_t kStaticScratchBytes = (size_t)8 << 20;   // 16 B per pair of channels: n_in * n_out up to 524288
static __device__ __align__(256) float scratch[kStaticScratchBytes / sizeof(float)];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
float *g_scratch_ptr[kMaxDevices] = {};
}  // namespace

size_t mix_static_scratch_bytes() { return kStaticScratchBytes; }

// 0, 10, 11 as launch_mix; 14 when the packed matrix does not fit the array
int launch_mix_static(float2 *r, const float2 *x, const float2 *w, long long rows, int n_in, int n_out, long long xs,
                      long long rs, bool adjoint, hipStream_t s) {
  if (rows == 0 || n_out == 0) return 0;
  if (mix_workspace_bytes(n_in, n_out) > kStaticScratchBytes) return 14;
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 10;
  float *ptr;
  {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
      float *p = nullptr;
      const hipError_t e = hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch));   // this device's copy
      if (e != hipSuccess || !p) return record_hip_error(e, "hipGetSymbolAddress(scratch)");
      g_scratch_ptr[dev] = p;
    }
    ptr = g_scratch_ptr[dev];
  }
  return launch_mix(r, x, w, rows, n_in, n_out, xs, rs, adjoint, ptr, kStaticScratchBytes, s);
}

// ---- gradient with respect to the matrix:  wg[c, o] = sum_rows conj(x[row, c]) g[row, o] ----------------------------------
// The reduction runs over the rows, hundreds of thousands of them, and the result is small.  In real terms
// D[kf][jf] = sum_rows xf[row][kf] gf[row][jf] over the floats of x and g as they lie in memory, and
// wg[c, o] = (D[2c][2o] + D[2c+1][2o+1]) + i (D[2c][2o+1] - D[2c+1][2o]).  One matrix instruction takes two rows:
// lane (i, h) supplies xf[row + h][.] and gf[row + h][.].  A lane loads EW consecutive floats of its row of x in one
// piece (the 64 lanes read 128 EW bytes of each of the two rows) and feeds them to EW instructions that add into EW
// separate 32 x 32 sums, so sum e of lane row i stands for kf = kf0 + EW i + e.  A wave owns 32 EW floats of x, JT
// tiles of 32 floats of g and a range of rows; the sums of the ranges go to a scratch array and a second kernel adds
// them in a fixed order and forms the complex result (no atomics: the result does not depend on timing).
struct WgradArgs {
  const float *x, *g;
  float *part;   // [nranges][k2][32 jt_total]
  long long rows, xs, gs, rows_per_range;
  int k2, n2, kgroups, jt_total;
};

template <int EW>
struct FloatVec;
template <>
struct FloatVec<4> { typedef float4 type; };
template <>
struct FloatVec<2> { typedef float2 type; };

template <int EW, int JT, int U>
struct WgradStage {
  typename FloatVec<EW>::type xv[U];
  float gv[U][JT];
};

template <int EW, int JT, int U>
__global__ void __launch_bounds__(64) wgrad_kernel(const WgradArgs p) {
  typedef typename FloatVec<EW>::type vec;
  const int lane = threadIdx.x, i = lane & 31, h = lane >> 5;
  const int kg = blockIdx.x % p.kgroups;
  const long long rr = blockIdx.x / p.kgroups;
  const int jt0 = blockIdx.y * JT;
  const int kf0 = kg * 32 * EW;
  int col = kf0 + EW * i;
  if (col > p.k2 - EW) col = p.k2 - EW;   // k2 is a multiple of 4: sums of columns past the end are not stored
  int jcol[JT];
#pragma unroll
  for (int c = 0; c < JT; c++) {
    jcol[c] = 32 * (jt0 + c) + i;
    if (jcol[c] > p.n2 - 1) jcol[c] = p.n2 - 1;
  }
  const long long r_begin = rr * p.rows_per_range;
  long long r_end = r_begin + p.rows_per_range;
  if (r_end > p.rows) r_end = p.rows;
  const float *xp = p.x + col;

  f16v acc[JT][EW];
#pragma unroll
  for (int c = 0; c < JT; c++)
#pragma unroll
    for (int e = 0; e < EW; e++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[c][e][v] = 0.f;

  // a row past the end of the range is read as the last row of the part and its g is replaced by zero when it is used
  auto load = [&](long long step, WgradStage<EW, JT, U> &st) {
#pragma unroll
    for (int u = 0; u < U; u++) {
      long long row = r_begin + step * (2 * U) + 2 * u + h;
      if (row > p.rows - 1) row = p.rows - 1;
      st.xv[u] = *(const vec *)(xp + row * p.xs);
#pragma unroll
      for (int c = 0; c < JT; c++) st.gv[u][c] = p.g[row * p.gs + jcol[c]];
    }
  };
  auto compute = [&](long long step, const WgradStage<EW, JT, U> &st) {
#pragma unroll
    for (int u = 0; u < U; u++) {
      const bool valid = r_begin + step * (2 * U) + 2 * u + h < r_end;
#pragma unroll
      for (int c = 0; c < JT; c++) {
        const float gv = valid ? st.gv[u][c] : 0.f;
        if constexpr (EW == 4) {
          acc[c][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(st.xv[u].x, gv, acc[c][0], 0, 0, 0);
          acc[c][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(st.xv[u].y, gv, acc[c][1], 0, 0, 0);
          acc[c][2] = __builtin_amdgcn_mfma_f32_32x32x2f32(st.xv[u].z, gv, acc[c][2], 0, 0, 0);
          acc[c][3] = __builtin_amdgcn_mfma_f32_32x32x2f32(st.xv[u].w, gv, acc[c][3], 0, 0, 0);
        } else {
          acc[c][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(st.xv[u].x, gv, acc[c][0], 0, 0, 0);
          acc[c][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(st.xv[u].y, gv, acc[c][1], 0, 0, 0);
        }
      }
    }
  };

  const long long nsteps = (r_end - r_begin + 2 * U - 1) / (2 * U);
  WgradStage<EW, JT, U> s0, s1;
  load(0, s0);
  long long q = 0;
  for (; q + 2 < nsteps; q += 2) {   // no branch inside, and fences: the next step's loads stay ahead of these sums
    load(q + 1, s1);
    __builtin_amdgcn_sched_barrier(0);
    compute(q, s0);
    __builtin_amdgcn_sched_barrier(0);
    load(q + 2, s0);
    __builtin_amdgcn_sched_barrier(0);
    compute(q + 1, s1);
    __builtin_amdgcn_sched_barrier(0);
  }
  if (q + 1 < nsteps) {
    load(q + 1, s1);
    compute(q, s0);
    compute(q + 1, s1);
  } else {
    compute(q, s0);
  }

  // register v of a sum holds row 8 (v / 4) + 4 h + (v % 4) of the 32 x 32 tile, column i
  const long long pitch = 32LL * p.jt_total;
  float *out = p.part + rr * p.k2 * pitch;
#pragma unroll
  for (int c = 0; c < JT; c++)
#pragma unroll
    for (int e = 0; e < EW; e++)
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int kf = kf0 + EW * (8 * (v / 4) + 4 * h + (v % 4)) + e;
        if (kf < p.k2) out[kf * pitch + 32 * (jt0 + c) + i] = acc[c][e][v];
      }
}

__global__ void __launch_bounds__(256) wgrad_sum_kernel(const float *part, float2 *wg, int n_in, int n_out, int nranges,
                                                        long long pitch) {
  const long long total = (long long)n_in * n_out;
  for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long long)gridDim.x * blockDim.x) {
    const int o = (int)(idx % n_out);
    const long long c = idx / n_out;
    float re = 0.f, im = 0.f;
    for (int r = 0; r < nranges; r++) {
      const float *d = part + ((long long)r * 2 * n_in + 2 * c) * pitch + 2 * o;
      re += d[0] + d[pitch + 1];
      im += d[1] - d[pitch];
    }
    wg[idx] = make_float2(re, im);
  }
}

namespace {
struct WgradPlan {
  int ew, jt, u, tiles, jt_total, kgroups;
  long long nranges, rows_per_range, pitch;
};
WgradPlan plan_wgrad(long long rows, int n_in, int n_out) {
  WgradPlan p;
  const int k2 = 2 * n_in, n2 = 2 * n_out;
  p.tiles = (n2 + 31) / 32;
  p.ew = p.tiles <= 2 ? 4 : 2;
  p.jt = p.tiles == 1 ? 1 : (p.tiles == 2 ? 2 : 4);
  p.u = p.tiles == 1 ? 16 : 8;
  p.jt_total = (p.tiles + p.jt - 1) / p.jt * p.jt;
  p.kgroups = (k2 + 32 * p.ew - 1) / (32 * p.ew);
  // enough waves to fill the chip a few times over, every range a whole number of steps and not empty
  const long long waves_per_range = (long long)p.kgroups * (p.jt_total / p.jt);
  long long nranges = std::max<long long>(1, std::min<long long>(4096 / waves_per_range, rows / (8LL * p.u)));
  nranges = std::min<long long>(nranges, 256);
  p.rows_per_range = ((rows + nranges - 1) / nranges + 2 * p.u - 1) / (2 * p.u) * (2 * p.u);
  p.nranges = (rows + p.rows_per_range - 1) / p.rows_per_range;
  p.pitch = 32LL * p.jt_total;
  return p;
}

__global__ void zero_fill_kernel(float2 *p, long long n) {
  for (long long i = blockIdx.x * 256LL + threadIdx.x; i < n; i += 256LL * gridDim.x) p[i] = make_float2(0.f, 0.f);
}
}  // namespace

// Bytes of workspace launch_mix_wgrad needs: the partial sums of the row ranges.
size_t mix_wgrad_workspace_bytes(long long rows, int n_in, int n_out) {
  if (rows <= 0 || n_in <= 0 || n_out <= 0) return 0;
  const WgradPlan p = plan_wgrad(rows, n_in, n_out);
  return sizeof(float) * (size_t)(p.nranges * 2 * n_in * p.pitch);
}

// 0, 10, 11 or 13 as launch_mix; the workspace (mix_wgrad_workspace_bytes) holds the partial sums of the row ranges
int launch_mix_wgrad(float2 *wg, const float2 *x, const float2 *g, long long rows, int n_in, int n_out, long long xs,
                     long long gs, float *ws, size_t ws_bytes, hipStream_t s) {
  if (n_in == 0 || n_out == 0) return 0;
  if ((n_in & 1) || (xs & 1) || ((uintptr_t)x & 15) || rows > (1LL << 38)) return 11;
  if (rows == 0) {   // a fill kernel, not a memset node: callers may capture this call into a graph
    const long long n = (long long)n_in * n_out;
    hipLaunchKernelGGL(zero_fill_kernel, dim3((unsigned)std::min<long long>((n + 255) / 256, 1024)), dim3(256), 0, s, wg, n);
    return hipGetLastError() == hipSuccess ? 0 : 10;
  }
  WgradArgs a;
  a.x = (const float *)x;
  a.g = (const float *)g;
  a.rows = rows;
  a.xs = 2 * xs;
  a.gs = 2 * gs;
  a.k2 = 2 * n_in;
  a.n2 = 2 * n_out;
  const WgradPlan pl = plan_wgrad(rows, n_in, n_out);
  const int tiles = pl.tiles, jt = pl.jt;
  a.jt_total = pl.jt_total;
  a.kgroups = pl.kgroups;
  a.rows_per_range = pl.rows_per_range;
  const long long nranges = pl.nranges, pitch = pl.pitch;
  if (!ws || ((uintptr_t)ws & 15) || ws_bytes < (size_t)(nranges * a.k2 * pitch) * sizeof(float)) return 13;
  float *part = ws;
  a.part = part;
  const dim3 grid((unsigned)(nranges * a.kgroups), (unsigned)(a.jt_total / jt));
  if (tiles == 1) hipLaunchKernelGGL((wgrad_kernel<4, 1, 16>), grid, dim3(64), 0, s, a);
  else if (tiles == 2) hipLaunchKernelGGL((wgrad_kernel<4, 2, 8>), grid, dim3(64), 0, s, a);
  else hipLaunchKernelGGL((wgrad_kernel<2, 4, 8>), grid, dim3(64), 0, s, a);
  const long long total = (long long)n_in * n_out;
  hipLaunchKernelGGL(wgrad_sum_kernel, dim3((unsigned)std::min<long long>((total + 255) / 256, 4096)), dim3(256), 0, s,
                     part, wg, n_in, n_out, (int)nranges, pitch);
  return hipGetLastError() == hipSuccess ? 0 : 10;
}

int mix_set_option(const char *name, int value) {   // 0, or 12 for a name that is not an option of this file
  if (std::string(name) == "mix_long") {
    g_mix_long = value;
    return 0;
  }
  if (std::string(name) == "mix_wide") {
    g_mix_wide = value;
    return 0;
  }
  if (std::string(name) == "mix_wide_waves") {
    g_mix_wide_waves = value;
    return 0;
  }
  if (std::string(name) == "mix_wide_store") {
    g_mix_wide_store = value;
    return 0;
  }
  return 12;
}

}  // namespace gelib_hip
