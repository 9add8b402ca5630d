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
// A wave owns 32 RT rows and CTW tiles of 32 output floats, and walks the reduction 32 floats (128 B of every row) at a
// time: lane (i, h) reads the 16 floats of its row that start at 16 h, so each row is read in whole 128-B lines.  V' is
// re-packed once per call into exactly the order the lanes read it (pack_kernel), 64 B per lane and step, and stays in L2.
// Bound: HBM for n_out <= 16 (8 B of x per 8 n_out flops is 16 flop/B at n_out = 16, below the fp32 matrix-core ridge of
// 157.3 TF / 8 TB/s = 19.7 flop/B), the matrix cores above that.
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
  const float *vp;   // packed V': [nq][ct_total][64 lanes][16] floats
  float *r;          // rows x (2 n_out) floats, row stride rs floats
  long long rows, xs, rs;
  int k2;            // 2 n_in
  int n2;            // 2 n_out
  int nq;            // ceil(k2 / 32)
  int ct_total;      // tiles of 32 output floats, padded to a multiple of CTW
};

// V'[kf][col] for kf = 2 P q + P h + j (j < P), col = 32 ct + i, stored at ((q * ct_total + ct) * 64 + lane) * P + j:
// P = 2^lg_p floats per lane and step, 16 for the short-step kernel and 64 for the long-step one
__global__ void __launch_bounds__(256) pack_kernel(const float2 *w, float *vp, int n_in, int n_out, int nq, int ct_total,
                                                   int adjoint, int lg_p) {
  const long long total = ((long long)nq * ct_total * 64) << lg_p;
  for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long long)gridDim.x * blockDim.x) {
    const int j = (int)(idx & ((1 << lg_p) - 1)), lane = (int)((idx >> lg_p) & 63);
    const long long tile = idx >> (lg_p + 6);
    const int ct = (int)(tile % ct_total), q = (int)(tile / ct_total);
    const int kf = ((2 * q + (lane >> 5)) << lg_p) + j, col = 32 * ct + (lane & 31);
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
  if (row0 >= p.rows) return;
  const int ct0 = blockIdx.y * CTW;
  const float *xrow[RT];
#pragma unroll
  for (int t = 0; t < RT; t++) {
    long long row = row0 + 32 * t + i;
    if (row > p.rows - 1) row = p.rows - 1;   // rows past the end repeat the last one; their results are not stored
    xrow[t] = p.x + row * p.xs + 16 * h;
  }
  const float *vp = p.vp + ((long long)ct0 * 64 + lane) * 16;
  const long long vstep = (long long)p.ct_total * 1024;

  // matrix instructions that add into the same registers run one after the other, so every wave keeps at least
  // four sums going: with fewer than four tiles the reduction is dealt over NCH sums per tile, added up at the end
  constexpr int NCH = RT * CTW >= 4 ? 1 : 4 / (RT * CTW);
  f16v acc[RT][CTW][NCH];
#pragma unroll
  for (int t = 0; t < RT; t++)
#pragma unroll
    for (int c = 0; c < CTW; c++)
#pragma unroll
      for (int n = 0; n < NCH; n++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[t][c][n][v] = 0.f;

  auto load = [&](int q, Operands<RT, CTW> &o) {
#pragma unroll
    for (int t = 0; t < RT; t++)
#pragma unroll
      for (int s = 0; s < 4; s++) {
        const int kf = 32 * q + 16 * h + 4 * s;   // k2 is a multiple of 4: a float4 is inside the row or outside it
        o.a[t][s] = kf < p.k2 ? *(const float4 *)(xrow[t] + 32 * q + 4 * s) : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
    for (int c = 0; c < CTW; c++)
#pragma unroll
      for (int s = 0; s < 4; s++) o.b[c][s] = *(const float4 *)(vp + q * vstep + c * 1024 + 4 * s);
  };
  auto compute = [&](const Operands<RT, CTW> &o) {
#pragma unroll
    for (int s = 0; s < 4; s++)
#pragma unroll
      for (int e = 0; e < 4; e++)
#pragma unroll
        for (int t = 0; t < RT; t++)
#pragma unroll
          for (int c = 0; c < CTW; c++) {
            const float av = e == 0 ? o.a[t][s].x : (e == 1 ? o.a[t][s].y : (e == 2 ? o.a[t][s].z : o.a[t][s].w));
            const float bv = e == 0 ? o.b[c][s].x : (e == 1 ? o.b[c][s].y : (e == 2 ? o.b[c][s].z : o.b[c][s].w));
            acc[t][c][e % NCH] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[t][c][e % NCH], 0, 0, 0);
          }
  };

  if (PIPE) {
    Operands<RT, CTW> o0, o1;
    load(0, o0);
    for (int q = 0; q < p.nq; q += 2) {
      if (q + 1 < p.nq) load(q + 1, o1);
      compute(o0);
      if (q + 1 < p.nq) {
        if (q + 2 < p.nq) load(q + 2, o0);
        compute(o1);
      }
    }
  } else {
    Operands<RT, CTW> o0;
    for (int q = 0; q < p.nq; q++) {
      load(q, o0);
      compute(o0);
    }
  }

  // register v of the 32 x 32 result holds row 8 (v / 4) + 4 h + (v % 4), column i
#pragma unroll
  for (int t = 0; t < RT; t++)
#pragma unroll
    for (int c = 0; c < CTW; c++) {
      const int col = 32 * (ct0 + c) + i;
      f16v sum = acc[t][c][0];
#pragma unroll
      for (int n = 1; n < NCH; n++) sum += acc[t][c][n];
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const long long row = row0 + 32 * t + 8 * (v / 4) + 4 * h + (v % 4);
        if (row < p.rows && col < p.n2) p.r[row * p.rs + col] = sum[v];
      }
    }
}

// Long reductions (n_in of hundreds or thousands).  In the kernel above a lane is tied to a row, so one load instruction
// touches 64 different cache lines and uses 16 B of each, and a row is visited 128 B at a time.  Here a wave of its own
// (a 64-thread block) reads 32 rows 512 B at a time with loads whose lanes run along the row (two rows per instruction),
// turns the tile through LDS into the layout of the matrix cores, and multiplies it while the loads of the next tile are
// in flight.  V' arrives 16 floats per lane at a time, one group ahead of the 16 matrix instructions that use it.
constexpr int kLongChunk = 128;            // floats of a row per step
constexpr int kLongPitch = kLongChunk + 4; // LDS row pitch: consecutive rows start 4 banks apart

template <int CTW>
__global__ void __launch_bounds__(64, 8) mix_long_kernel(const MixArgs p) {
  __shared__ float4 tile4[32 * kLongPitch / 4];
  float *tile = (float *)tile4;
  const int lane = threadIdx.x, i = lane & 31, h = lane >> 5;
  const long long groups = (p.rows + 31) / 32;
  const long long grp = blockIdx.x % groups;
  const int ct0 = (int)(blockIdx.x / groups) * CTW;
  const long long row0 = grp * 32;

  // loads: instruction u covers rows 2u and 2u+1, lane (i, h) the 16 bytes at float 4 i of row 2u + h
  long long lrow = row0 + h;
  const float *src[16];
#pragma unroll
  for (int u = 0; u < 16; u++) {
    long long row = lrow + 2 * u;
    if (row > p.rows - 1) row = p.rows - 1;   // rows past the end repeat the last one; their results are not stored
    src[u] = p.x + row * p.xs + 4 * i;
  }
  const float *vp = p.vp + ((long long)ct0 * 64 + lane) * 64;
  const long long vstep = (long long)p.ct_total * 4096;

  constexpr int NCH = CTW >= 4 ? 1 : 4 / CTW;   // sums per tile, as in the kernel above
  f16v acc[CTW][NCH];
#pragma unroll
  for (int c = 0; c < CTW; c++)
#pragma unroll
    for (int n = 0; n < NCH; n++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[c][n][v] = 0.f;

  float4 stage[16];
  auto fetch = [&](int q) {
    const bool inside = q * kLongChunk + 4 * i < p.k2;   // k2 is a multiple of 4
#pragma unroll
    for (int u = 0; u < 16; u++)
      stage[u] = inside ? *(const float4 *)(src[u] + q * kLongChunk) : make_float4(0.f, 0.f, 0.f, 0.f);
  };
  fetch(0);
  for (int q = 0; q < p.nq; q++) {
    __syncthreads();   // the reads of the previous tile are over
#pragma unroll
    for (int u = 0; u < 16; u++) *(float4 *)(tile + (2 * u + h) * kLongPitch + 4 * i) = stage[u];
    __syncthreads();
    float4 a[16];
#pragma unroll
    for (int s = 0; s < 16; s++) a[s] = *(const float4 *)(tile + i * kLongPitch + 64 * h + 4 * s);
    if (q + 1 < p.nq) fetch(q + 1);
    const float *vq = vp + q * vstep;
    float4 b[2][4];
#pragma unroll
    for (int s = 0; s < 4; s++) b[0][s] = *(const float4 *)(vq + 4 * s);
#pragma unroll
    for (int g = 0; g < 4 * CTW; g++) {   // group g: output tile g / 4, floats 16 (g % 4) .. of the lane's 64
      if (g + 1 < 4 * CTW) {
#pragma unroll
        for (int s = 0; s < 4; s++)
          b[(g + 1) & 1][s] = *(const float4 *)(vq + ((g + 1) / 4) * 4096 + 16 * ((g + 1) % 4) + 4 * s);
      }
#pragma unroll
      for (int s = 0; s < 4; s++) {
        const float4 av = a[4 * (g % 4) + s], bv = b[g & 1][s];
        f16v *sum = acc[g / 4];
        sum[0 % NCH] = __builtin_amdgcn_mfma_f32_32x32x2f32(av.x, bv.x, sum[0 % NCH], 0, 0, 0);
        sum[1 % NCH] = __builtin_amdgcn_mfma_f32_32x32x2f32(av.y, bv.y, sum[1 % NCH], 0, 0, 0);
        sum[2 % NCH] = __builtin_amdgcn_mfma_f32_32x32x2f32(av.z, bv.z, sum[2 % NCH], 0, 0, 0);
        sum[3 % NCH] = __builtin_amdgcn_mfma_f32_32x32x2f32(av.w, bv.w, sum[3 % NCH], 0, 0, 0);
      }
    }
  }

#pragma unroll
  for (int c = 0; c < CTW; c++) {
    const int col = 32 * (ct0 + c) + i;
    f16v sum = acc[c][0];
#pragma unroll
    for (int n = 1; n < NCH; n++) sum += acc[c][n];
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const long long row = row0 + 8 * (v / 4) + 4 * h + (v % 4);
      if (row < p.rows && col < p.n2) p.r[row * p.rs + col] = sum[v];
    }
  }
}

// the packed matrix of a call lives in a buffer kept per (device, stream): calls on one stream are ordered, calls on
// different streams do not share a buffer
struct Workspace {
  float *ptr = nullptr;
  size_t bytes = 0;
};
std::mutex g_ws_mutex;
std::map<std::pair<int, hipStream_t>, Workspace> g_ws;

float *workspace(size_t bytes, hipStream_t s) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return nullptr;
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  Workspace &w = g_ws[{dev, s}];
  if (w.bytes < bytes) {
    if (w.ptr) {
      if (hipStreamSynchronize(s) != hipSuccess) return nullptr;   // an earlier call on this stream may still read it
      (void)hipFree(w.ptr);
      w.ptr = nullptr;
      w.bytes = 0;
    }
    const size_t want = std::max(bytes, (size_t)1 << 20);
    if (hipMalloc((void **)&w.ptr, want) != hipSuccess) return nullptr;
    w.bytes = want;
  }
  return w.ptr;
}

int g_mix_long = 1;

template <int RT, int CTW, bool PIPE>
void launch(const MixArgs &a, hipStream_t s) {
  const long long waves = (a.rows + 32 * RT - 1) / (32 * RT);
  dim3 grid((unsigned)((waves + 3) / 4), (unsigned)(a.ct_total / CTW));
  hipLaunchKernelGGL((mix_kernel<RT, CTW, PIPE>), grid, dim3(256), 0, s, a);
}

}  // namespace

// 0 on success, 10 when a HIP call fails, 11 when the shape is not one this kernel takes (n_in odd, strides that break
// the 16-byte alignment of a row)
int launch_mix(float2 *r, const float2 *x, const float2 *w, long long rows, int n_in, int n_out, long long xs,
               long long rs, bool adjoint, hipStream_t s) {
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
  const int tiles = (a.n2 + 31) / 32;
  const bool long_rows = a.k2 >= 4 * kLongChunk && g_mix_long;   // rows of 2 KB and more: the LDS-staged kernel
  const bool wide = tiles > 2;
  const int ctw = wide ? 4 : tiles;
  a.ct_total = (tiles + ctw - 1) / ctw * ctw;
  const int lg_p = long_rows ? 6 : 4;
  a.nq = (a.k2 + (2 << lg_p) - 1) / (2 << lg_p);
  const long long total = ((long long)a.nq * a.ct_total * 64) << lg_p;
  float *vp = workspace((size_t)total * sizeof(float), s);
  if (!vp) return 10;
  a.vp = vp;
  hipLaunchKernelGGL(pack_kernel, dim3((unsigned)std::min<long long>((total + 255) / 256, 4096)), dim3(256), 0, s, w, vp,
                     n_in, n_out, a.nq, a.ct_total, adjoint ? 1 : 0, lg_p);
  if (long_rows) {
    const long long blocks = (rows + 31) / 32 * (a.ct_total / ctw);
    if (blocks > 0x7fffffffLL) return 11;
    if (ctw == 1) hipLaunchKernelGGL(mix_long_kernel<1>, dim3((unsigned)blocks), dim3(64), 0, s, a);
    else if (ctw == 2) hipLaunchKernelGGL(mix_long_kernel<2>, dim3((unsigned)blocks), dim3(64), 0, s, a);
    else hipLaunchKernelGGL(mix_long_kernel<4>, dim3((unsigned)blocks), dim3(64), 0, s, a);
  } else if (!wide) {
    if (ctw == 1) launch<2, 1, true>(a, s);
    else launch<2, 2, true>(a, s);
  } else if (a.nq <= 2) {
    launch<2, 4, false>(a, s);
  } else {
    launch<1, 4, true>(a, s);
  }
  return hipGetLastError() == hipSuccess ? 0 : 10;
}

int mix_set_option(const char *name, int value) {   // 0, or 12 for a name that is not an option of this file
  if (std::string(name) == "mix_long") {
    g_mix_long = value;
    return 0;
  }
  return 12;
}

}  // namespace gelib_hip
