// C ABI of libgelib_hip.so: argument validation, broadcasting, triple enumeration and kernel selection.
//
// The validation mirrors what the reference checks on the way to its launchers -- the dispatcher's batch/grid
// reconciliation (core/CGproduct.hpp:44-104, core/Gpart.hpp:168-185, 416-432) and the launcher's own tests
// (cuda/SO3part_addCGproduct.cu:189-214) -- but reports a status code instead of printing and skipping.
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <functional>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "cg_common.h"
#include "cg_linear.h"
#include "cg_staged.h"
#include "cg_unrolled.h"

using namespace gelib_hip;

namespace gelib_hip {

namespace {
thread_local std::string t_last_error;
thread_local int t_last_path = kPathNone;
int g_force_generic = 0;
int g_check_pointers = 1;
}  // namespace

int record_hip_error(hipError_t e, const char *what) {
  t_last_error = std::string(what) + ": " + hipGetErrorString(e);
  (void)hipGetLastError();  // clear the sticky error so that later calls are not blamed for it
  return GELIB_HIP_ERR_RUNTIME;
}

namespace {
void forget_ranges(const void *base);
struct ScratchBuf {
  char *ptr = nullptr;
  size_t bytes = 0;
};
constexpr int kScratchKinds = 2;
std::mutex g_scratch_mutex[kScratchKinds];
std::map<std::pair<int, hipStream_t>, ScratchBuf> g_scratch[kScratchKinds];
// memory the caller has lent for a stream (gelib_hip_set_stream_workspace): kind k uses the k-th of kScratchKinds equal
// slices.  It is the caller's to keep alive, so it also serves calls that are being recorded into a graph.
std::mutex g_lent_mutex;
std::map<std::pair<int, hipStream_t>, ScratchBuf> g_lent;
}  // namespace

std::mutex &stream_scratch_mutex(int kind) { return g_scratch_mutex[kind]; }

int stream_scratch(int kind, hipStream_t s, size_t bytes, void **out) {
  *out = nullptr;
  int dev = 0;
  GELIB_HIP_TRY(hipGetDevice(&dev));
  {
    std::lock_guard<std::mutex> lock(g_lent_mutex);
    auto it = g_lent.find({dev, s});
    if (it != g_lent.end()) {
      const size_t slice = (it->second.bytes / kScratchKinds) & ~(size_t)255;
      if (bytes <= slice) {
        *out = it->second.ptr + (size_t)kind * slice;
        return GELIB_HIP_OK;
      }
    }
  }
  // A call that is being recorded into a graph gets none of the library's own (*out = nullptr) and takes its
  // scratch-free route: the graph would keep the buffer's address, and a later call that needs a larger buffer frees it.
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &cap) != hipSuccess) (void)hipGetLastError();
  if (cap != hipStreamCaptureStatusNone) return GELIB_HIP_OK;
  ScratchBuf &buf = g_scratch[kind][{dev, s}];
  if (buf.bytes < bytes) {
    if (buf.ptr) {
      forget_ranges(buf.ptr);
      GELIB_HIP_TRY(hipFree(buf.ptr));  // waits for the kernels that still use it
    }
    buf.ptr = nullptr;
    buf.bytes = 0;
    GELIB_HIP_TRY(hipMalloc((void **)&buf.ptr, bytes));
    buf.bytes = bytes;
  }
  *out = buf.ptr;
  return GELIB_HIP_OK;
}

namespace {

struct View {  // one validated descriptor
  const gelib_part_desc *d;
  int l;
  int n;
};

int check_desc(const gelib_part_desc *d, View &v) {
  if (!d) return GELIB_HIP_ERR_NULL;
  for (int k = 0; k < 5; k++)
    if (d->dims[k] < 0 || d->strides[k] < 0) return GELIB_HIP_ERR_ARG;   // whatever "check_pointers" says
  if (d->dims[3] % 2 != 1) return GELIB_HIP_ERR_ODD_DIM;
  if (d->dims[3] > 2 * (4 * kMaxL) + 1 || d->dims[4] > 0x7fffffffLL) return GELIB_HIP_ERR_PARTS;
  v.d = d;
  v.l = (int)(d->dims[3] - 1) / 2;
  v.n = (int)d->dims[4];
  const bool empty = d->dims[0] == 0 || d->dims[1] == 0 || d->dims[2] == 0 || d->dims[4] == 0;
  if (!d->ptr && !empty) return GELIB_HIP_ERR_NULL;
  return GELIB_HIP_OK;
}

// Allocations that have passed the driver's checks: [base, base + size) on a device.  A view that lies inside one of
// them passes without any driver call (a product call checks 15 to 30 pointers, most of them in the same few
// allocations of a caching allocator, call after call).  An entry lives until it is pushed out by newer ones; memory
// that is freed and handed out again by the driver at the same address as a different kind is not noticed, which is
// the price of not asking every time ("check_pointers" 2 asks every time).
struct KnownRange {
  const char *base;
  size_t size;
  int device;
};
constexpr int kKnownRanges = 64;
std::mutex g_known_mutex;
KnownRange g_known[kKnownRanges];
int g_known_count = 0, g_known_next = 0;

bool known_range(const char *p, const char *end, int dev) {
  std::lock_guard<std::mutex> lock(g_known_mutex);
  for (int i = 0; i < g_known_count; i++)
    if (g_known[i].device == dev && p >= g_known[i].base && end <= g_known[i].base + g_known[i].size) return true;
  return false;
}

// base == nullptr: forget everything; otherwise the entries that start at base (the allocation is being freed)
void forget_ranges(const void *base) {
  std::lock_guard<std::mutex> lock(g_known_mutex);
  int k = 0;
  for (int i = 0; i < g_known_count; i++)
    if (base && g_known[i].base != (const char *)base) g_known[k++] = g_known[i];
  g_known_count = k;
  g_known_next = k % kKnownRanges;
}

void remember_range(const char *base, size_t size, int dev) {
  std::lock_guard<std::mutex> lock(g_known_mutex);
  g_known[g_known_next] = {base, size, dev};
  g_known_next = (g_known_next + 1) % kKnownRanges;
  if (g_known_count < kKnownRanges) g_known_count++;
}

// The farthest element of the view must lie inside the allocation that holds ptr, and that allocation must be
// device (or managed) memory: a host pointer or an over-long view would otherwise fault the GPU.
int check_range(const void *ptr, const int64_t dims[5], const int64_t strides[5], size_t elem_bytes) {
  if (!g_check_pointers || !ptr) return GELIB_HIP_OK;
  long long span = 0;
  for (int k = 0; k < 5; k++) {
    if (dims[k] == 0) return GELIB_HIP_OK;
    if (strides[k] < 0) return GELIB_HIP_ERR_ARG;
    span += (dims[k] - 1) * strides[k];
  }
  const char *end = (const char *)ptr + (span + 1) * (long long)elem_bytes;
  int dev = 0;
  const bool have_dev = hipGetDevice(&dev) == hipSuccess;   // no driver call: the runtime keeps it per thread
  if (g_check_pointers == 1 && have_dev && known_range((const char *)ptr, end, dev)) return GELIB_HIP_OK;
  hipPointerAttribute_t attr;
  hipError_t e = hipPointerGetAttributes(&attr, ptr);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return GELIB_HIP_ERR_DEVICE;
  }
  if (attr.type != hipMemoryTypeDevice && attr.type != hipMemoryTypeManaged) return GELIB_HIP_ERR_DEVICE;
  if (have_dev && attr.type == hipMemoryTypeDevice && attr.device != dev) return GELIB_HIP_ERR_DEVICE;
  hipDeviceptr_t base = nullptr;
  size_t size = 0;
  e = hipMemGetAddressRange(&base, &size, (hipDeviceptr_t)ptr);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return GELIB_HIP_OK;  // range unknown (e.g. a suballocator the runtime cannot see): type check above stands
  }
  if (end > (const char *)base + size) return GELIB_HIP_ERR_DEVICE;
  if (have_dev) remember_range((const char *)base, size, dev);
  return GELIB_HIP_OK;
}

int check_pointer(const gelib_part_desc *d) { return check_range(d->ptr, d->dims, d->strides, sizeof(float2)); }

PartDev to_dev(const gelib_part_desc *d, const long long E[3], long long own[3]) {
  PartDev p;
  p.ptr = (float2 *)d->ptr;
  long long s[3];
  for (int k = 0; k < 3; k++) {
    own[k] = (d->dims[k] == E[k]) ? E[k] : 1;
    s[k] = (d->dims[k] == E[k] && E[k] > 1) ? d->strides[k] : 0;
  }
  p.sb = s[0];
  p.sg0 = s[1];
  p.sg1 = s[2];
  p.sm = d->strides[3];
  p.sc = d->strides[4];
  return p;
}

// A destination whose view repeats memory (extent > 1 with stride 0, e.g. an expanded torch view) would be written by
// many threads at once; a destination that is to be summed over a dimension has extent 1 there instead.
int check_dest(const gelib_part_desc *d) {
  for (int k = 0; k < 5; k++)
    if (d->dims[k] > 1 && d->strides[k] == 0) return GELIB_HIP_ERR_BROADCAST_DEST;
  return GELIB_HIP_OK;
}

// dims equal or 1 along each leading dimension; dimension 0 is the batch, 1..2 the grid
int reconcile(const gelib_part_desc *const *ds, int n, long long E[3]) {
  for (int k = 0; k < 3; k++) {
    long long e = 1;
    bool zero = false;
    for (int i = 0; i < n; i++) {
      if (ds[i]->dims[k] == 0) zero = true;
      e = std::max(e, (long long)ds[i]->dims[k]);
    }
    if (zero) e = 0;
    for (int i = 0; i < n; i++)
      if (ds[i]->dims[k] != e && ds[i]->dims[k] != 1) return k == 0 ? GELIB_HIP_ERR_BATCH : GELIB_HIP_ERR_GRID;
    E[k] = e;
  }
  return GELIB_HIP_OK;
}

// roles: r = product/gradient, x = first operand (or its gradient), y = second operand (or its gradient)
int make_part_op(const gelib_part_desc *r, const gelib_part_desc *x, const gelib_part_desc *y, int offs, bool diag,
                 PartOp &op) {
  View vr, vx, vy;
  int rc;
  if ((rc = check_desc(r, vr))) return rc;
  if ((rc = check_desc(x, vx))) return rc;
  if ((rc = check_desc(y, vy))) return rc;
  if (vx.l > kMaxL || vy.l > kMaxL) return GELIB_HIP_ERR_PARTS;
  if (vr.l < std::abs(vx.l - vy.l) || vr.l > vx.l + vy.l) return GELIB_HIP_ERR_TRIANGLE;
  if (diag && vx.n != vy.n) return GELIB_HIP_ERR_DIAG_CHANNELS;
  if (offs < 0) return GELIB_HIP_ERR_ARG;
  const long long nout = diag ? vx.n : (long long)vx.n * vy.n;
  if (nout > 0x7fffffffLL || offs + nout > vr.n) return GELIB_HIP_ERR_CHANNELS;
  const gelib_part_desc *ds[3] = {r, x, y};
  if ((rc = reconcile(ds, 3, op.E))) return rc;
  op.r = to_dev(r, op.E, op.Dr);
  op.x = to_dev(x, op.E, op.Dx);
  op.y = to_dev(y, op.E, op.Dy);
  op.l1 = vx.l;
  op.l2 = vy.l;
  op.l = vr.l;
  op.n1 = vx.n;
  op.n2 = vy.n;
  op.nout = (int)nout;
  op.offs = offs;
  op.diag = diag;
  return GELIB_HIP_OK;
}


// ---- gradient destinations that broadcast ---------------------------------------------------------------------
// A gradient whose destination has extent 1 where the operation has extent E (the operand is shared by the batch or by
// the grid, core/Gpart.hpp:168-185) is a sum over that dimension.  The product kernels then write one gradient per
// cell into a packed temporary and bcast_reduce.hip adds those up in a fixed order; the batch is taken in chunks so
// that the temporary stays within "bcast_scratch_kb" KiB (64 MiB unless set) (it is 1 % of the bytes of g at the headline type).  The
// temporary belongs to the library: one buffer per (device, stream), allocated by the first such call and grown when a
// later one needs more.
int g_bcast_scratch_kb = 64 * 1024;
int g_bcast_reduce = 1;

bool dest_broadcasts(const gelib_part_desc *d, const long long E[3]) {
  for (int k = 0; k < 3; k++)
    if (d->dims[k] == 1 && E[k] > 1) return true;
  return false;
}

// descs: the descriptors of the call (copies the caller's `inner` reads); dests: indices of the destinations among
// them; inner(accumulate) runs the operation on descs as they stand.
int with_bcast_dests(std::vector<gelib_part_desc> &descs, const std::vector<int> &dests, const long long E[3],
                     int accumulate, hipStream_t s, const std::function<int(int)> &inner) {
  const std::vector<gelib_part_desc> orig = descs;
  std::vector<int> bidx;
  bool all_bcast = true;
  for (int i : dests) {
    if (dest_broadcasts(&orig[i], E)) bidx.push_back(i);
    else all_bcast = false;
  }
  const long long G = E[1] * E[2];
  long long per_cell = 0;
  for (int i : bidx) per_cell += orig[i].dims[3] * orig[i].dims[4] * (long long)sizeof(float2);
  if (per_cell == 0 || E[0] * G == 0) return inner(accumulate);
  const long long cap = (long long)std::max(1, g_bcast_scratch_kb) << 10;
  const long long cb = std::max<long long>(1, std::min<long long>(E[0], cap / std::max<long long>(1, per_cell * G)));
  if (cb * G > 0x7fffffffLL) return GELIB_HIP_ERR_ARG;
  const long long Ec[3] = {cb, E[1], E[2]};
  size_t partial = 0;
  for (int i : bidx) {
    const long long D[3] = {orig[i].dims[0] == 1 ? 1 : cb, orig[i].dims[1] == 1 ? 1 : E[1], orig[i].dims[2] == 1 ? 1 : E[2]};
    partial = std::max(partial, bcast_partial_bytes(Ec, D, (int)orig[i].dims[3], (int)orig[i].dims[4]));
  }
  const size_t tmp_bytes = ((size_t)(cb * G * per_cell) + 255) & ~(size_t)255;
  const size_t need = tmp_bytes + partial;
  // held while the kernels of this call are put on the stream: another thread using the same stream's buffer must
  // come entirely before or entirely after them
  std::lock_guard<std::mutex> lock(stream_scratch_mutex(0));
  struct {
    char *ptr;
  } buf;
  int rc = stream_scratch(0, s, need, (void **)&buf.ptr);
  if (rc) return rc;
  if (!buf.ptr) return GELIB_HIP_ERR_UNSUPPORTED;  // under stream capture: the caller sums inside the shape-agnostic kernels
  for (long long b0 = 0; b0 < E[0]; b0 += cb) {
    const long long cbn = std::min(cb, E[0] - b0);
    const long long En[3] = {cbn, E[1], E[2]};
    for (size_t i = 0; i < descs.size(); i++) {
      descs[i] = orig[i];
      if (orig[i].dims[0] == E[0] && E[0] > 1) {
        descs[i].ptr = (char *)orig[i].ptr + b0 * orig[i].strides[0] * (long long)sizeof(float2);
        descs[i].dims[0] = cbn;
      }
    }
    size_t off = 0;
    for (int i : bidx) {
      gelib_part_desc &d = descs[i];
      const long long rows = orig[i].dims[3], n = orig[i].dims[4];
      d.ptr = buf.ptr + off;
      d.dims[0] = cbn, d.dims[1] = E[1], d.dims[2] = E[2];
      d.strides[4] = 1, d.strides[3] = n, d.strides[2] = rows * n, d.strides[1] = E[2] * rows * n;
      d.strides[0] = G * rows * n;
      off += (size_t)(cb * G * rows * n) * sizeof(float2);
    }
    const int inner_acc = (accumulate && !all_bcast) ? 1 : 0;
    if (inner_acc)
      for (int i : bidx) {
        long long own[3];
        PartDev pd = to_dev(&descs[i], En, own);
        if ((rc = launch_zero_fill(pd, own, (int)descs[i].dims[3], (int)descs[i].dims[4], s))) return rc;
      }
    if ((rc = inner(inner_acc))) return rc;
    for (int i : bidx) {
      gelib_part_desc d = orig[i];
      if (orig[i].dims[0] == E[0] && E[0] > 1) {
        d.ptr = (char *)orig[i].ptr + b0 * orig[i].strides[0] * (long long)sizeof(float2);
        d.dims[0] = cbn;
      }
      long long own[3];
      PartDev pd = to_dev(&d, En, own);
      const bool summed_over_batch = orig[i].dims[0] == 1 && E[0] > 1;
      rc = launch_bcast_reduce((const float2 *)descs[i].ptr, (float2 *)(buf.ptr + tmp_bytes), pd, En, own,
                               (int)d.dims[3], (int)d.dims[4], accumulate != 0 || (summed_over_batch && b0 > 0), s);
      if (rc) return rc;
    }
  }
  return GELIB_HIP_OK;
}

enum Kind { kFwd, kBack0, kBack1 };

int part_entry(Kind kind, bool diag, const gelib_part_desc *r, const gelib_part_desc *x, const gelib_part_desc *y,
               int offs, int accumulate, void *stream) {
  t_last_path = kPathNone;
  PartOp op;
  int rc = make_part_op(r, x, y, offs, diag, op);
  if (rc) return rc;
  if ((rc = check_dest(kind == kFwd ? r : (kind == kBack0 ? x : y)))) return rc;
  if ((rc = check_pointer(r)) || (rc = check_pointer(x)) || (rc = check_pointer(y))) return rc;
  if (op.E[0] * op.E[1] * op.E[2] == 0 || op.nout == 0) return GELIB_HIP_OK;
  hipStream_t s = (hipStream_t)stream;
  if (!g_force_generic && g_bcast_reduce && kind != kFwd && dest_broadcasts(kind == kBack0 ? x : y, op.E)) {
    std::vector<gelib_part_desc> d = {*r, *x, *y};
    rc = with_bcast_dests(d, {kind == kBack0 ? 1 : 2}, op.E, accumulate, s, [&](int acc) {
      return part_entry(kind, diag, &d[0], &d[1], &d[2], offs, acc, stream);
    });
    if (rc != GELIB_HIP_ERR_UNSUPPORTED) return rc;
    t_last_path = kPathGeneric;   // no scratch (the call is being recorded into a graph): the serial sum
    return kind == kBack0 ? launch_generic_back0(op, accumulate != 0, s) : launch_generic_back1(op, accumulate != 0, s);
  }
  if (!g_force_generic) {
    int used = 0;
    if (diag && kind == kFwd) {
      // One lane per channel beats the lane-per-channel-pair kernels for a Diag product going forward.  Backward, a single
      // triple keeps one of the four waves of the Diag kernel's blocks busy and the other families win (1.3 vs 1.5 ms
      // at l = 4, 64 channels, 131072 cells), so the gradients of one triple stay with them.
      rc = diag6_part(0, op.E, r, x, y, op.l1, op.l2, op.l, offs, accumulate != 0, s, &used);
      if (rc) return rc;
      if (used) {
        t_last_path = kPathDiag6;
        return GELIB_HIP_OK;
      }
    }
    rc = unrolled_part(kind == kFwd ? 0 : (kind == kBack0 ? 1 : 2), op, accumulate != 0, s, &used);
    if (rc) return rc;
    if (used) {
      t_last_path = kPathUnrolled;
      return GELIB_HIP_OK;
    }
    rc = staged_part(kind == kFwd ? 0 : (kind == kBack0 ? 1 : 2), op, accumulate != 0, s, &used);
    if (rc) return rc;
    if (used) {
      t_last_path = kPathStaged;
      return GELIB_HIP_OK;
    }
  }
  t_last_path = kPathGeneric;
  switch (kind) {
    case kFwd: return launch_generic_fwd(op, accumulate != 0, s);
    case kBack0: return launch_generic_back0(op, accumulate != 0, s);
    case kBack1: return launch_generic_back1(op, accumulate != 0, s);
  }
  return GELIB_HIP_ERR_ARG;
}

// ---- SO3vec level ---------------------------------------------------------------------------------------------

int sort_parts(int n, const gelib_part_desc *parts, int max_parts, std::vector<View> &out) {
  if (n < 0 || n > max_parts) return GELIB_HIP_ERR_PARTS;
  if (n > 0 && !parts) return GELIB_HIP_ERR_NULL;
  out.resize(n);
  for (int i = 0; i < n; i++) {
    int rc = check_desc(&parts[i], out[i]);
    if (rc) return rc;
  }
  std::sort(out.begin(), out.end(), [](const View &a, const View &b) { return a.l < b.l; });
  for (int i = 1; i < n; i++)
    if (out[i].l == out[i - 1].l) return GELIB_HIP_ERR_PARTS;
  return GELIB_HIP_OK;
}

// check_channels = false: the parts of R only say which l are wanted (the fused product -> mixing entry, whose
// destination has the mixing's output channels, not the product's)
int build_vec_plan(bool diag, const std::vector<View> &R, const std::vector<View> &X, const std::vector<View> &Y,
                   VecPlan &plan, bool check_channels = true) {
  for (auto &v : X)
    if (v.l > kMaxL) return GELIB_HIP_ERR_PARTS;
  for (auto &v : Y)
    if (v.l > kMaxL) return GELIB_HIP_ERR_PARTS;
  std::vector<const gelib_part_desc *> all;
  for (auto &v : R) all.push_back(v.d);
  for (auto &v : X) all.push_back(v.d);
  for (auto &v : Y) all.push_back(v.d);
  int rc = reconcile(all.data(), (int)all.size(), plan.E);
  if (rc) return rc;
  plan.diag = diag;
  plan.triples.clear();
  std::vector<long long> offset(2 * (2 * kMaxL) + 2, 0);
  for (int p = 0; p < (int)X.size(); p++)
    for (int q = 0; q < (int)Y.size(); q++) {
      const int l1 = X[p].l, l2 = Y[q].l;
      for (int l = std::abs(l1 - l2); l <= l1 + l2; l++) {
        int k = -1;
        for (int t = 0; t < (int)R.size(); t++)
          if (R[t].l == l) k = t;
        if (k < 0) continue;  // absent product part: skipped, offsets of other parts unaffected
        if (diag && X[p].n != Y[q].n) return GELIB_HIP_ERR_DIAG_CHANNELS;
        const long long nout = diag ? X[p].n : (long long)X[p].n * Y[q].n;
        if (check_channels && offset[l] + nout > R[k].n) return GELIB_HIP_ERR_CHANNELS;
        if (offset[l] + nout > 0x7fffffffLL) return GELIB_HIP_ERR_CHANNELS;
        plan.triples.push_back({p, q, k, l1, l2, l, (int)offset[l], (int)nout});
        offset[l] += nout;
      }
    }
  return GELIB_HIP_OK;
}

PartOp triple_op(const VecPlan &plan, const VecTriple &t, const std::vector<View> &R, const std::vector<View> &X,
                 const std::vector<View> &Y) {
  PartOp op;
  for (int d = 0; d < 3; d++) op.E[d] = plan.E[d];
  op.r = to_dev(R[t.ri].d, op.E, op.Dr);
  op.x = to_dev(X[t.xi].d, op.E, op.Dx);
  op.y = to_dev(Y[t.yi].d, op.E, op.Dy);
  op.l1 = t.l1;
  op.l2 = t.l2;
  op.l = t.l;
  op.n1 = X[t.xi].n;
  op.n2 = Y[t.yi].n;
  op.nout = t.nout;
  op.offs = t.offs;
  op.diag = plan.diag;
  return op;
}

// A Diag product that reaches above l = 6: the lane-per-channel kernels (built for products up to l = 6) take the
// triples up to there, the other families the rest.  R is sorted by l, so A keeps a prefix of it and B the remainder.
// (A CGproduct with a one-channel operand is such a Diag product with the channel repeated, and is split the same way.)
bool split_at_l6(const VecPlan &plan, const std::vector<View> &R, VecPlan &A, VecPlan &B, std::vector<View> &RA,
                 std::vector<View> &RB);
bool split_diag(const VecPlan &plan, const std::vector<View> &R, const std::vector<View> &X, const std::vector<View> &Y,
                VecPlan &A, VecPlan &B, std::vector<View> &RA, std::vector<View> &RB, bool forward = false) {
  if (!plan.diag) {
    auto all_one = [](const std::vector<View> &v) {
      for (auto &p : v)
        if (p.n != 1) return false;
      return true;
    };
    const bool nx = all_one(X), ny = all_one(Y);
    // exactly one narrow side; forward also one channel on both sides (the Diag product of one channel)
    if (nx == ny && !(forward && nx)) return false;
  }
  return split_at_l6(plan, R, A, B, RA, RB);
}

// The triples of a plan up to l = 6 (A, with the parts RA) and above (B, RB); false when one of the two is empty.
bool split_at_l6(const VecPlan &plan, const std::vector<View> &R, VecPlan &A, VecPlan &B, std::vector<View> &RA,
                 std::vector<View> &RB) {
  constexpr int kSplit = 6;
  bool lo = false, hi = false;
  for (auto &t : plan.triples) (t.l <= kSplit ? lo : hi) = true;
  if (!lo || !hi) return false;
  size_t k0 = 0;
  while (k0 < R.size() && R[k0].l <= kSplit) k0++;
  A.diag = B.diag = plan.diag;
  for (int k = 0; k < 3; k++) A.E[k] = B.E[k] = plan.E[k];
  for (auto t : plan.triples) {
    if (t.l <= kSplit) {
      A.triples.push_back(t);
    } else {
      t.ri -= (int)k0;
      B.triples.push_back(t);
    }
  }
  RA.assign(R.begin(), R.begin() + k0);
  RB.assign(R.begin() + k0, R.end());
  return true;
}

int g_pairwise = 1;  // vectors of several parts with l above 7: one launch of the single-pair kernels per pair

// The kernel families in the order they are tried, then the shape-agnostic kernels.
int fwd_dispatch(const VecPlan &plan, const std::vector<View> &R, const std::vector<View> &X, const std::vector<View> &Y,
                 int accumulate, hipStream_t s) {
  int rc;
  if (!g_force_generic) {
    std::vector<const gelib_part_desc *> rd, xd, yd;
    for (auto &v : R) rd.push_back(v.d);
    for (auto &v : X) xd.push_back(v.d);
    for (auto &v : Y) yd.push_back(v.d);
    int used = 0;
    // Diag products: one lane per channel beats the lane-per-channel-pair kernels
    rc = diag6_vec_fwd(plan, rd, xd, yd, accumulate != 0, s, &used);
    if (rc) return rc;
    if (used) {
      t_last_path = kPathDiag6;
      return GELIB_HIP_OK;
    }
    rc = unrolled_vec_fwd(plan, rd, xd, yd, accumulate != 0, s, &used);
    if (rc) return rc;
    if (used) {
      t_last_path = kPathUnrolled;
      return GELIB_HIP_OK;
    }
    {
      // A CGproduct of operands above l = 4 that reaches above l = 6 (the API default is uncapped): the unrolled kernel
      // built for such operands takes the triples up to l = 6, the any-l kernels the rest (different product parts).
      int lop = 0;
      for (auto &v : X) lop = std::max(lop, v.l);
      for (auto &v : Y) lop = std::max(lop, v.l);
      VecPlan A, B;
      std::vector<View> RA, RB;
      if (!plan.diag && lop > 4 && lop <= 6 && split_at_l6(plan, R, A, B, RA, RB)) {
        std::vector<const gelib_part_desc *> ra;
        for (auto &v : RA) ra.push_back(v.d);
        rc = unrolled_vec_fwd(A, ra, xd, yd, accumulate != 0, s, &used);
        if (rc) return rc;
        if (used) {
          rc = fwd_dispatch(B, RB, X, Y, accumulate, s);
          t_last_path = kPathUnrolled;
          return rc;
        }
      }
    }
    rc = onepair_mfma_vec_fwd(plan, rd, xd, yd, accumulate != 0, s, &used);
    if (rc) return rc;
    if (used) {
      t_last_path = kPathOnePair;
      return GELIB_HIP_OK;
    }
    {
      // Vectors of several parts with l above 7: one launch of the matrix-core single-pair kernel per (x part, y part)
      // pair (every pair writes channel blocks of its own); a pair that kernel does not take goes through this
      // dispatch by itself.
      int lop = 0;
      for (auto &v : X) lop = std::max(lop, v.l);
      for (auto &v : Y) lop = std::max(lop, v.l);
      if (g_pairwise && !plan.diag && X.size() * Y.size() >= 2 && lop > 7) {
        bool any = false;
        for (int p = 0; p < (int)X.size(); p++)
          for (int q = 0; q < (int)Y.size(); q++) {
            VecPlan sub;
            sub.diag = plan.diag;
            for (int k = 0; k < 3; k++) sub.E[k] = plan.E[k];
            for (auto t : plan.triples)
              if (t.xi == p && t.yi == q) {
                t.xi = t.yi = 0;
                sub.triples.push_back(t);
              }
            if (sub.triples.empty()) continue;
            rc = onepair_mfma_vec_fwd(sub, rd, {X[p].d}, {Y[q].d}, accumulate != 0, s, &used);
            if (rc) return rc;
            if (used) any = true;
            else if (!any) goto whole;  // not even the first pair: the vector stays in one piece
            else if ((rc = fwd_dispatch(sub, R, {X[p]}, {Y[q]}, accumulate, s))) return rc;
          }
        if (any) {
          t_last_path = kPathOnePair;
          return GELIB_HIP_OK;
        }
      }
    }
  whole:
    {
      rc = staged_vec_fwd(plan, rd, xd, yd, accumulate != 0, s, &used);
      if (rc) return rc;
      if (used) {
        t_last_path = kPathStaged;
        return GELIB_HIP_OK;
      }
    }
  }
  t_last_path = kPathGeneric;
  for (auto &t : plan.triples) {
    PartOp op = triple_op(plan, t, R, X, Y);
    if ((rc = launch_generic_fwd(op, accumulate != 0, s))) return rc;
  }
  return GELIB_HIP_OK;
}

int vec_fwd_entry(bool diag, int nr, const gelib_part_desc *r, int nx, const gelib_part_desc *x, int ny,
                  const gelib_part_desc *y, int accumulate, void *stream) {
  t_last_path = kPathNone;
  std::vector<View> R, X, Y;
  int rc;
  if ((rc = sort_parts(nr, r, kMaxOutParts, R)) || (rc = sort_parts(nx, x, kMaxParts, X)) ||
      (rc = sort_parts(ny, y, kMaxParts, Y)))
    return rc;
  if (R.empty() || X.empty() || Y.empty()) return GELIB_HIP_OK;
  VecPlan plan;
  if ((rc = build_vec_plan(diag, R, X, Y, plan))) return rc;
  for (auto &v : R)
    if ((rc = check_dest(v.d))) return rc;
  for (auto &v : R)
    if ((rc = check_pointer(v.d))) return rc;
  for (auto &v : X)
    if ((rc = check_pointer(v.d))) return rc;
  for (auto &v : Y)
    if ((rc = check_pointer(v.d))) return rc;
  if (plan.E[0] * plan.E[1] * plan.E[2] == 0 || plan.triples.empty()) return GELIB_HIP_OK;
  hipStream_t s = (hipStream_t)stream;
  if (!g_force_generic) {
    VecPlan A, B;
    std::vector<View> RA, RB;
    if (split_diag(plan, R, X, Y, A, B, RA, RB, true)) {
      std::vector<const gelib_part_desc *> rd, xd, yd;
      for (auto &v : RA) rd.push_back(v.d);
      for (auto &v : X) xd.push_back(v.d);
      for (auto &v : Y) yd.push_back(v.d);
      int used = 0;
      if ((rc = diag6_vec_fwd(A, rd, xd, yd, accumulate != 0, s, &used))) return rc;
      if (used) {
        rc = fwd_dispatch(B, RB, X, Y, accumulate, s);
        t_last_path = kPathDiag6;
        return rc;
      }
    }
  }
  return fwd_dispatch(plan, R, X, Y, accumulate, s);
}

// Vectors of several parts with l above 7: one launch of the single-pair kernels per (x part, y part) pair, each adding
// its share to the two gradient parts it touches (launches on one stream run one after the other, so the order of the
// additions is fixed).  The any-l kernels would otherwise take such vectors in one pass that adds partial sums into LDS
// with float atomics; g is read once either way.  Taken only when every pair is one the single-pair kernels accept.
int pairwise_onepair_bwd(const VecPlan &plan, const std::vector<View> &G, const std::vector<View> &X,
                         const std::vector<View> &Y, const std::vector<View> &XG, const std::vector<View> &YG,
                         const std::vector<const gelib_part_desc *> &gd, bool want_x, bool want_y, int accumulate,
                         hipStream_t s, int *used) {
  *used = 0;
  if (!g_pairwise || !want_x || !want_y || X.size() * Y.size() < 2) return GELIB_HIP_OK;
  int lop = 0;
  for (auto &v : X) lop = std::max(lop, v.l);
  for (auto &v : Y) lop = std::max(lop, v.l);
  if (g_pairwise == 1 && lop <= 7) return GELIB_HIP_OK;   // the striped kernels (fixed order, no atomics) take those
  struct Sub {
    VecPlan plan;
    int p, q;
  };
  std::vector<Sub> subs;
  for (int p = 0; p < (int)X.size(); p++)
    for (int q = 0; q < (int)Y.size(); q++) {
      Sub sub;
      sub.p = p;
      sub.q = q;
      sub.plan.diag = plan.diag;
      for (int k = 0; k < 3; k++) sub.plan.E[k] = plan.E[k];
      for (auto t : plan.triples)
        if (t.xi == p && t.yi == q) {
          t.xi = t.yi = 0;
          sub.plan.triples.push_back(t);
        }
      if (!sub.plan.triples.empty()) subs.push_back(sub);
    }
  if (subs.empty()) return GELIB_HIP_OK;
  int rc;
  for (auto &sub : subs) {  // first pass: would every pair be taken?
    int ok = 0;
    if ((rc = onepair_vec_bwd(sub.plan, gd, {X[sub.p].d}, {Y[sub.q].d}, {XG[sub.p].d}, {YG[sub.q].d}, true, s, &ok, true)))
      return rc;
    if (!ok) return GELIB_HIP_OK;
  }
  if (!accumulate) {  // every pair adds; a part that no pair feeds is still written (zeros)
    for (auto *L : {&XG, &YG})
      for (auto &v : *L) {
        long long own[3];
        PartDev pd = to_dev(v.d, plan.E, own);
        if ((rc = launch_zero_fill(pd, own, 2 * v.l + 1, v.n, s))) return rc;
      }
  }
  for (auto &sub : subs) {
    int ok = 0;
    const std::vector<const gelib_part_desc *> x1 = {X[sub.p].d}, y1 = {Y[sub.q].d}, xg1 = {XG[sub.p].d}, yg1 = {YG[sub.q].d};
    if ((rc = onepair_mfma_vec_bwd(sub.plan, gd, x1, y1, xg1, yg1, true, s, &ok))) return rc;
    if (!ok && (rc = onepair_vec_bwd(sub.plan, gd, x1, y1, xg1, yg1, true, s, &ok))) return rc;
    if (!ok) return GELIB_HIP_ERR_ARG;  // cannot happen: the first pass asked
  }
  *used = 1;
  return GELIB_HIP_OK;
}

int bwd_dispatch(const VecPlan &plan, const std::vector<View> &G, const std::vector<View> &X, const std::vector<View> &Y,
                 const std::vector<View> &XG, const std::vector<View> &YG, bool want_x, bool want_y, int accumulate,
                 hipStream_t s, bool skip_unrolled = false) {
  int rc;
  if (!g_force_generic && !plan.triples.empty()) {
    std::vector<const gelib_part_desc *> gd, xd, yd, xgd, ygd;
    for (auto &v : G) gd.push_back(v.d);
    for (auto &v : X) xd.push_back(v.d);
    for (auto &v : Y) yd.push_back(v.d);
    for (auto &v : XG) xgd.push_back(v.d);
    for (auto &v : YG) ygd.push_back(v.d);
    int used = 0;
    rc = diag6_vec_bwd(plan, gd, xd, yd, xgd, ygd, accumulate != 0, s, &used);
    if (rc) return rc;
    if (used) {
      t_last_path = kPathDiag6;
      return GELIB_HIP_OK;
    }
    if (!skip_unrolled) {
      rc = unrolled_vec_bwd(plan, gd, xd, yd, xgd, ygd, accumulate != 0, s, &used);
      if (rc) return rc;
      if (used) {
        t_last_path = kPathUnrolled;
        return GELIB_HIP_OK;
      }
    }
    rc = onepair_mfma_vec_bwd(plan, gd, xd, yd, xgd, ygd, accumulate != 0, s, &used);
    if (rc) return rc;
    if (used) {
      t_last_path = kPathOnePair;
      return GELIB_HIP_OK;
    }
    rc = onepair_vec_bwd(plan, gd, xd, yd, xgd, ygd, accumulate != 0, s, &used);
    if (rc) return rc;
    if (used) {
      t_last_path = kPathOnePair;
      return GELIB_HIP_OK;
    }
    rc = pairwise_onepair_bwd(plan, G, X, Y, XG, YG, gd, want_x, want_y, accumulate, s, &used);
    if (rc) return rc;
    if (used) {
      t_last_path = kPathOnePair;
      return GELIB_HIP_OK;
    }
    rc = staged_vec_bwd(plan, gd, xd, yd, xgd, ygd, accumulate != 0, s, &used);
    if (rc) return rc;
    if (used) {
      t_last_path = kPathStaged;
      return GELIB_HIP_OK;
    }
  }
  t_last_path = kPathGeneric;
  // shape-agnostic route: zero the destinations when overwriting, then one accumulation per triple,
  // all back0 first and then all back1 like the reference (python/src/gelib/SO3vec.py:267-268)
  if (!accumulate) {
    for (auto *L : {&XG, &YG})
      for (auto &v : *L) {
        long long own[3];
        PartDev pd = to_dev(v.d, plan.E, own);
        if ((rc = launch_zero_fill(pd, own, 2 * v.l + 1, v.n, s))) return rc;
      }
  }
  if (want_x)
    for (auto &t : plan.triples) {
      PartOp op = triple_op(plan, t, G, XG, Y);
      if ((rc = launch_generic_back0(op, true, s))) return rc;
    }
  if (want_y)
    for (auto &t : plan.triples) {
      PartOp op = triple_op(plan, t, G, X, YG);
      if ((rc = launch_generic_back1(op, true, s))) return rc;
    }
  return GELIB_HIP_OK;
}

int vec_bwd_entry(bool diag, const gelib_part_desc *xg, const gelib_part_desc *yg, int ng, const gelib_part_desc *g,
                  int nx, const gelib_part_desc *x, int ny, const gelib_part_desc *y, int accumulate, void *stream) {
  t_last_path = kPathNone;
  if (!xg && !yg) return GELIB_HIP_OK;
  std::vector<View> G, X, Y, XG, YG;
  int rc;
  if ((rc = sort_parts(ng, g, kMaxOutParts, G)) || (rc = sort_parts(nx, x, kMaxParts, X)) ||
      (rc = sort_parts(ny, y, kMaxParts, Y)))
    return rc;
  if (xg && (rc = sort_parts(nx, xg, kMaxParts, XG))) return rc;
  if (yg && (rc = sort_parts(ny, yg, kMaxParts, YG))) return rc;
  // gradients are shaped like their operands (l and channel count; leading dimensions may broadcast)
  for (int i = 0; xg && i < nx; i++)
    if (XG[i].l != X[i].l || XG[i].n != X[i].n) return GELIB_HIP_ERR_PARTS;
  for (int i = 0; yg && i < ny; i++)
    if (YG[i].l != Y[i].l || YG[i].n != Y[i].n) return GELIB_HIP_ERR_PARTS;
  if (G.empty() || X.empty() || Y.empty()) return GELIB_HIP_OK;
  VecPlan plan;
  if ((rc = build_vec_plan(diag, G, X, Y, plan))) return rc;
  {  // the gradients take part in the batch/grid reconciliation too
    std::vector<const gelib_part_desc *> all;
    for (auto &v : G) all.push_back(v.d);
    for (auto &v : X) all.push_back(v.d);
    for (auto &v : Y) all.push_back(v.d);
    for (auto &v : XG) all.push_back(v.d);
    for (auto &v : YG) all.push_back(v.d);
    if ((rc = reconcile(all.data(), (int)all.size(), plan.E))) return rc;
  }
  for (auto *L : {&XG, &YG})
    for (auto &v : *L)
      if ((rc = check_dest(v.d))) return rc;
  for (auto *L : {&G, &X, &Y, &XG, &YG})
    for (auto &v : *L)
      if ((rc = check_pointer(v.d))) return rc;
  if (plan.E[0] * plan.E[1] * plan.E[2] == 0) return GELIB_HIP_OK;
  hipStream_t s = (hipStream_t)stream;
  if (!g_force_generic && g_bcast_reduce) {
    bool bcast = false;
    for (auto *L : {&XG, &YG})
      for (auto &v : *L) bcast = bcast || dest_broadcasts(v.d, plan.E);
    if (bcast) {
      // descriptors in the caller's order: g, x, y, xg, yg
      std::vector<gelib_part_desc> d;
      d.insert(d.end(), g, g + ng);
      d.insert(d.end(), x, x + nx);
      d.insert(d.end(), y, y + ny);
      const int ixg = (int)d.size();
      if (xg) d.insert(d.end(), xg, xg + nx);
      const int iyg = (int)d.size();
      if (yg) d.insert(d.end(), yg, yg + ny);
      std::vector<int> dests;
      for (int i = ixg; i < (int)d.size(); i++) dests.push_back(i);
      rc = with_bcast_dests(d, dests, plan.E, accumulate, s, [&](int acc) {
        return vec_bwd_entry(diag, xg ? &d[ixg] : nullptr, yg ? &d[iyg] : nullptr, ng, &d[0], nx, &d[ng], ny, &d[ng + nx],
                             acc, stream);
      });
      if (rc != GELIB_HIP_ERR_UNSUPPORTED) return rc;
      // no scratch (the call is being recorded into a graph): the families below decline a destination that
      // broadcasts, and the shape-agnostic kernels sum it serially
    }
  }
  if (!g_force_generic) {
    VecPlan A, B;
    std::vector<View> GA, GB;
    if (split_diag(plan, G, X, Y, A, B, GA, GB)) {
      std::vector<const gelib_part_desc *> gd, xd, yd, xgd, ygd;
      for (auto &v : GA) gd.push_back(v.d);
      for (auto &v : X) xd.push_back(v.d);
      for (auto &v : Y) yd.push_back(v.d);
      for (auto &v : XG) xgd.push_back(v.d);
      for (auto &v : YG) ygd.push_back(v.d);
      int used = 0;
      if ((rc = diag6_vec_bwd(A, gd, xd, yd, xgd, ygd, accumulate != 0, s, &used))) return rc;
      if (used) {
        // The rest adds on top of what the first part wrote.  It is a few triples of a vector with many parts: the
        // unrolled backward kernels stage and flush the images of all parts per cell whatever the number of triples
        // (39 ms against 18 ms on Diag L=4, 64 channels, 131072 cells, uncapped), so they are passed over here.
        rc = bwd_dispatch(B, GB, X, Y, XG, YG, xg != nullptr, yg != nullptr, 1, s, true);
        t_last_path = kPathDiag6;
        return rc;
      }
    }
  }
  return bwd_dispatch(plan, G, X, Y, XG, YG, xg != nullptr, yg != nullptr, accumulate, s);
}

// Channels of the product's parts (indexed like R) for a plan built with check_channels = false.
std::vector<long long> product_channels(const VecPlan &plan, size_t nparts) {
  std::vector<long long> tau(nparts, 0);
  for (auto &t : plan.triples) tau[t.ri] = std::max(tau[t.ri], (long long)t.offs + t.nout);
  return tau;
}

int linear_fwd_entry(int nr, const gelib_part_desc *r, int nx, const gelib_part_desc *x, int ny,
                     const gelib_part_desc *y, const void *const *w, int accumulate, void *workspace,
                     uint64_t workspace_bytes, void *stream) {
  t_last_path = kPathNone;
  std::vector<View> R, X, Y;
  int rc;
  if ((rc = sort_parts(nr, r, kMaxOutParts, R)) || (rc = sort_parts(nx, x, kMaxParts, X)) ||
      (rc = sort_parts(ny, y, kMaxParts, Y)))
    return rc;
  if (R.empty() || X.empty() || Y.empty()) return GELIB_HIP_OK;
  if (!w) return GELIB_HIP_ERR_NULL;
  VecPlan plan;
  if ((rc = build_vec_plan(false, R, X, Y, plan, false))) return rc;
  const std::vector<long long> tau = product_channels(plan, R.size());
  std::vector<const float2 *> W(R.size());
  for (size_t k = 0; k < R.size(); k++) {
    W[k] = (const float2 *)w[R[k].d - r];
    if (tau[k] > 0 && R[k].n > 0 && !W[k]) return GELIB_HIP_ERR_NULL;
  }
  for (auto &v : R)
    if ((rc = check_dest(v.d))) return rc;
  for (auto &v : R)
    if ((rc = check_pointer(v.d))) return rc;
  for (auto &v : X)
    if ((rc = check_pointer(v.d))) return rc;
  for (auto &v : Y)
    if ((rc = check_pointer(v.d))) return rc;
  for (size_t k = 0; k < R.size(); k++) {
    if (tau[k] == 0 || R[k].n == 0) continue;
    const int64_t wd[5] = {tau[k], 1, 1, 1, R[k].n}, wst[5] = {R[k].n, 0, 0, 0, 1};
    if ((rc = check_range(W[k], wd, wst, 2 * sizeof(float)))) return rc;
  }
  const int64_t sd[5] = {(int64_t)workspace_bytes, 1, 1, 1, 1}, sst[5] = {1, 0, 0, 0, 0};
  if (workspace && workspace_bytes && (rc = check_range(workspace, sd, sst, 1))) return rc;
  if (plan.E[0] * plan.E[1] * plan.E[2] == 0) return GELIB_HIP_OK;
  std::vector<const gelib_part_desc *> rd, xd, yd;
  for (auto &v : R) rd.push_back(v.d);
  for (auto &v : X) xd.push_back(v.d);
  for (auto &v : Y) yd.push_back(v.d);
  int used = 0;
  rc = cg_linear_fwd(plan, rd, xd, yd, W, accumulate != 0, workspace, (size_t)workspace_bytes, (hipStream_t)stream, &used);
  if (rc) return rc;
  if (!used) return GELIB_HIP_ERR_UNSUPPORTED;
  t_last_path = kPathLinear;
  return GELIB_HIP_OK;
}


// ---- backward of CGproduct followed by the weight matrices, in bounded memory ------------------------------------
// out_l = P_l W_l with P = CGproduct(x, y):  xg, yg = the product's backward pass on gP_l = gout_l W_l^H, and
// wg_l = sum over the rows of P_l^H gout_l.  Neither P nor gP is ever held at full size: the batch is taken in chunks
// whose product fits the caller's workspace; a chunk's product is formed by the forward kernels, read by the
// matrix-gradient kernel, overwritten in place by gP and read once more by the backward kernels.
struct LinBwdShape {
  std::vector<View> G, X, Y, XG, YG;
  VecPlan plan;
  std::vector<long long> tau;     // channels of the product's parts, indexed like G
  long long rows_per_batch = 0;   // sum over l of grid cells * (2l+1)
  long long G01 = 1;              // grid cells per batch entry
};

size_t lin_bwd_bytes(const LinBwdShape &sh, long long cb, size_t *p_bytes, size_t *mix_bytes, size_t *wg_ws_bytes,
                     size_t *wg_tmp_bytes) {
  size_t pb = 0, mb = 0, wb = 0, tb = 0;
  for (size_t k = 0; k < sh.G.size(); k++) {
    const long long rows = cb * sh.G01 * (2 * sh.G[k].l + 1);
    pb += (((size_t)rows * sh.tau[k] * sizeof(float2)) + 255) & ~(size_t)255;
    mb = std::max(mb, mix_workspace_bytes(sh.G[k].n, (int)sh.tau[k]));
    wb = std::max(wb, mix_wgrad_workspace_bytes(rows, (int)sh.tau[k], sh.G[k].n));
    tb = std::max(tb, (size_t)sh.tau[k] * sh.G[k].n * sizeof(float2));
  }
  auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
  if (p_bytes) *p_bytes = pb;
  if (mix_bytes) *mix_bytes = up(mb);
  if (wg_ws_bytes) *wg_ws_bytes = up(wb);
  if (wg_tmp_bytes) *wg_tmp_bytes = up(tb);
  return pb + up(mb) + up(wb) + up(tb);
}

// validation shared by the size query and the call; g: the gradient of the output (nr parts, n_out_l channels)
int lin_bwd_shape(int ng, const gelib_part_desc *g, int nx, const gelib_part_desc *x, int ny, const gelib_part_desc *y,
                  const gelib_part_desc *xg, const gelib_part_desc *yg, LinBwdShape &sh) {
  int rc;
  if ((rc = sort_parts(ng, g, kMaxOutParts, sh.G)) || (rc = sort_parts(nx, x, kMaxParts, sh.X)) ||
      (rc = sort_parts(ny, y, kMaxParts, sh.Y)))
    return rc;
  if (xg && (rc = sort_parts(nx, xg, kMaxParts, sh.XG))) return rc;
  if (yg && (rc = sort_parts(ny, yg, kMaxParts, sh.YG))) return rc;
  for (size_t i = 0; i < sh.XG.size(); i++)
    if (sh.XG[i].l != sh.X[i].l || sh.XG[i].n != sh.X[i].n) return GELIB_HIP_ERR_PARTS;
  for (size_t i = 0; i < sh.YG.size(); i++)
    if (sh.YG[i].l != sh.Y[i].l || sh.YG[i].n != sh.Y[i].n) return GELIB_HIP_ERR_PARTS;
  if (sh.G.empty() || sh.X.empty() || sh.Y.empty()) return GELIB_HIP_ERR_UNSUPPORTED;
  if ((rc = build_vec_plan(false, sh.G, sh.X, sh.Y, sh.plan, false))) return rc;
  {
    std::vector<const gelib_part_desc *> all;
    for (auto *L : {&sh.G, &sh.X, &sh.Y, &sh.XG, &sh.YG})
      for (auto &v : *L) all.push_back(v.d);
    if ((rc = reconcile(all.data(), (int)all.size(), sh.plan.E))) return rc;
  }
  sh.tau = product_channels(sh.plan, sh.G.size());
  sh.G01 = sh.plan.E[1] * sh.plan.E[2];
  // what the matrix kernels need: every tensor with the full leading extents, gout packed so that its rows (cell, m) are
  // one stride apart, even channel counts on both sides of every matrix
  for (auto *L : {&sh.G, &sh.X, &sh.Y, &sh.XG, &sh.YG})
    for (auto &v : *L)
      for (int k = 0; k < 3; k++)
        if (v.d->dims[k] != sh.plan.E[k]) return GELIB_HIP_ERR_UNSUPPORTED;
  for (size_t k = 0; k < sh.G.size(); k++) {
    const gelib_part_desc *d = sh.G[k].d;
    const long long rows_cell = 2 * sh.G[k].l + 1;
    if (d->strides[4] != 1 || (d->strides[3] & 1) || d->strides[3] < d->dims[4]) return GELIB_HIP_ERR_UNSUPPORTED;
    if (d->dims[2] > 1 && d->strides[2] != rows_cell * d->strides[3]) return GELIB_HIP_ERR_UNSUPPORTED;
    if (d->dims[1] > 1 && d->strides[1] != d->dims[2] * rows_cell * d->strides[3]) return GELIB_HIP_ERR_UNSUPPORTED;
    if (d->dims[0] > 1 && d->strides[0] != d->dims[1] * d->dims[2] * rows_cell * d->strides[3]) return GELIB_HIP_ERR_UNSUPPORTED;
    if (((uintptr_t)d->ptr & 15) || (sh.G[k].n & 1) || (sh.tau[k] & 1) || sh.tau[k] == 0 || sh.G[k].n == 0 ||
        sh.tau[k] > 0x7fffffffLL)
      return GELIB_HIP_ERR_UNSUPPORTED;
  }
  return GELIB_HIP_OK;
}

int linear_bwd_entry(const gelib_part_desc *xg, const gelib_part_desc *yg, void *const *wg, int ng,
                     const gelib_part_desc *g, int nx, const gelib_part_desc *x, int ny, const gelib_part_desc *y,
                     const void *const *w, int accumulate, void *workspace, uint64_t workspace_bytes, void *stream) {
  t_last_path = kPathNone;
  if (!xg && !yg && !wg) return GELIB_HIP_OK;
  if (!w) return GELIB_HIP_ERR_NULL;
  LinBwdShape sh;
  int rc = lin_bwd_shape(ng, g, nx, x, ny, y, xg, yg, sh);
  if (rc) return rc;
  for (auto *L : {&sh.XG, &sh.YG})
    for (auto &v : *L)
      if ((rc = check_dest(v.d))) return rc;
  for (auto *L : {&sh.G, &sh.X, &sh.Y, &sh.XG, &sh.YG})
    for (auto &v : *L)
      if ((rc = check_pointer(v.d))) return rc;
  std::vector<const float2 *> W(sh.G.size());
  std::vector<float2 *> WG(sh.G.size(), nullptr);
  for (size_t k = 0; k < sh.G.size(); k++) {
    const size_t orig = sh.G[k].d - g;   // position in the caller's order, which w and wg follow
    W[k] = (const float2 *)w[orig];
    if (wg) WG[k] = (float2 *)wg[orig];
    if (!W[k] || (wg && !WG[k])) return GELIB_HIP_ERR_NULL;
    const int64_t wd[5] = {sh.tau[k], 1, 1, 1, sh.G[k].n}, wst[5] = {sh.G[k].n, 0, 0, 0, 1};
    if ((rc = check_range(W[k], wd, wst, 2 * sizeof(float)))) return rc;
    if (wg && (rc = check_range(WG[k], wd, wst, 2 * sizeof(float)))) return rc;
  }
  const long long E0 = sh.plan.E[0];
  if (E0 * sh.G01 == 0) return GELIB_HIP_OK;
  if (!workspace || ((uintptr_t)workspace & 255)) return GELIB_HIP_ERR_WORKSPACE;
  const int64_t sd[5] = {(int64_t)workspace_bytes, 1, 1, 1, 1}, sst[5] = {1, 0, 0, 0, 0};
  if ((rc = check_range(workspace, sd, sst, 1))) return rc;
  // the largest chunk of the batch whose product fits the workspace
  long long cb = E0;
  while (cb > 1 && lin_bwd_bytes(sh, cb, nullptr, nullptr, nullptr, nullptr) > workspace_bytes) cb = (cb + 1) / 2;
  size_t pb, mb, wb, tb;
  if (lin_bwd_bytes(sh, cb, &pb, &mb, &wb, &tb) > workspace_bytes) return GELIB_HIP_ERR_WORKSPACE;
  char *base = (char *)workspace;
  float *mix_ws = (float *)(base + pb), *wg_ws = (float *)(base + pb + mb);
  float2 *wg_tmp = (float2 *)(base + pb + mb + wb);
  hipStream_t s = (hipStream_t)stream;

  auto chunk_of = [&](const gelib_part_desc &d, long long b0, long long cbn) {
    gelib_part_desc c = d;
    c.ptr = (char *)d.ptr + b0 * d.strides[0] * (long long)sizeof(float2);
    c.dims[0] = cbn;
    return c;
  };
  for (long long b0 = 0; b0 < E0; b0 += cb) {
    const long long cbn = std::min(cb, E0 - b0);
    std::vector<gelib_part_desc> P(sh.G.size()), gc(ng), xc(nx), yc(ny), xgc, ygc;
    for (int i = 0; i < ng; i++) gc[i] = chunk_of(g[i], b0, cbn);
    for (int i = 0; i < nx; i++) xc[i] = chunk_of(x[i], b0, cbn);
    for (int i = 0; i < ny; i++) yc[i] = chunk_of(y[i], b0, cbn);
    if (xg) for (int i = 0; i < nx; i++) xgc.push_back(chunk_of(xg[i], b0, cbn));
    if (yg) for (int i = 0; i < ny; i++) ygc.push_back(chunk_of(yg[i], b0, cbn));
    size_t off = 0;
    for (size_t k = 0; k < sh.G.size(); k++) {   // the chunk's product parts, packed
      const long long rows_cell = 2 * sh.G[k].l + 1, n = sh.tau[k];
      gelib_part_desc &d = P[k];
      d.ptr = base + off;
      d.dims[0] = cbn, d.dims[1] = sh.plan.E[1], d.dims[2] = sh.plan.E[2], d.dims[3] = rows_cell, d.dims[4] = n;
      d.strides[4] = 1, d.strides[3] = n, d.strides[2] = rows_cell * n, d.strides[1] = sh.plan.E[2] * rows_cell * n;
      d.strides[0] = sh.G01 * rows_cell * n;
      off += (((size_t)cb * sh.G01 * rows_cell * n * sizeof(float2)) + 255) & ~(size_t)255;
    }
    // 1. the chunk's product
    if ((rc = vec_fwd_entry(false, (int)P.size(), P.data(), nx, xc.data(), ny, yc.data(), 0, stream))) return rc;
    for (size_t k = 0; k < sh.G.size(); k++) {
      const gelib_part_desc &go = gc[sh.G[k].d - g];
      const long long rows = cbn * sh.G01 * (2 * sh.G[k].l + 1);
      const int tau = (int)sh.tau[k], n_out = sh.G[k].n;
      // 2. gradient of the matrix: first chunk straight into wg (or onto it), later chunks through the temporary
      if (wg) {
        const bool direct = b0 == 0 && !accumulate;
        rc = launch_mix_wgrad(direct ? WG[k] : wg_tmp, (const float2 *)P[k].ptr, (const float2 *)go.ptr, rows, tau, n_out,
                              tau, go.strides[3], wg_ws, wb, s);
        if (rc) return rc == 11 ? GELIB_HIP_ERR_UNSUPPORTED : rc;
        if (!direct && (rc = launch_add_into(WG[k], wg_tmp, (long long)tau * n_out, true, s))) return rc;
      }
      // 3. gradient of the product, over the product itself
      if (xg || yg) {
        rc = launch_mix((float2 *)P[k].ptr, (const float2 *)go.ptr, W[k], rows, n_out, tau, go.strides[3], tau, true, mix_ws,
                        mb, s);
        if (rc) return rc == 11 ? GELIB_HIP_ERR_UNSUPPORTED : rc;
      }
    }
    // 4. the product's backward pass on it
    if (xg || yg) {
      rc = vec_bwd_entry(false, xg ? xgc.data() : nullptr, yg ? ygc.data() : nullptr, (int)P.size(), P.data(), nx, xc.data(),
                         ny, yc.data(), accumulate, stream);
      if (rc) return rc;
    }
  }
  return GELIB_HIP_OK;
}

}  // namespace
}  // namespace gelib_hip

extern "C" {

const char *gelib_hip_strerror(int status) {
  switch (status) {
    case GELIB_HIP_OK: return "ok";
    case GELIB_HIP_ERR_NULL: return "null descriptor or data pointer";
    case GELIB_HIP_ERR_ODD_DIM: return "dimension -2 of an SO3part must be odd (2l+1)";
    case GELIB_HIP_ERR_TRIANGLE: return "|l1-l_2| <= l <= l1+l2 not satisfied";
    case GELIB_HIP_ERR_DIAG_CHANNELS: return "DiagCGproduct needs equal channel counts (N1==N2)";
    case GELIB_HIP_ERR_CHANNELS: return "fragment dimension of r not large enough";
    case GELIB_HIP_ERR_BATCH: return "batch dimensions cannot be reconciled";
    case GELIB_HIP_ERR_GRID: return "grid dimensions cannot be reconciled";
    case GELIB_HIP_ERR_DEVICE: return "SO3part must be on GPU (pointer is not device memory of the current device, or the view overruns its allocation)";
    case GELIB_HIP_ERR_PARTS: return "too many parts, a repeated l, l above the supported maximum, or gradient parts that do not match their operand";
    case GELIB_HIP_ERR_RUNTIME: return "HIP runtime error";
    case GELIB_HIP_ERR_BROADCAST_DEST: return "the destination repeats memory (a dimension of extent > 1 with stride 0)";
    case GELIB_HIP_ERR_ARG: return "malformed argument";
    case GELIB_HIP_ERR_WORKSPACE: return "workspace missing, not 16-byte aligned or too small";
    case GELIB_HIP_ERR_TOO_LARGE:
      return "the packed matrix of n_in x n_out channels exceeds the 8 MiB array of the entry point that allocates "
             "nothing; use gelib_hip_part_mix_channels with a workspace";
    case GELIB_HIP_ERR_UNSUPPORTED:
      return "shapes outside what the fused kernel takes; form the product and mix its channels in two calls";
  }
  return "unknown status";
}

const char *gelib_hip_last_runtime_error(void) { return t_last_error.c_str(); }

const char *gelib_hip_version(void) { return "gelib_hip 0.1 (gfx950)"; }

int gelib_hip_cg_matrix(int l1, int l2, int l, float *out) {
  if (!out) return GELIB_HIP_ERR_NULL;
  if (l1 < 0 || l2 < 0 || l < std::abs(l1 - l2) || l > l1 + l2) return GELIB_HIP_ERR_TRIANGLE;
  cg_matrix_host(l1, l2, l, out);
  return GELIB_HIP_OK;
}

int gelib_hip_so3type_product(int diag, int nx, const int *lx, const int *cx, int ny, const int *ly, const int *cy,
                              int maxl, int64_t *n_out, int len) {
  if ((nx > 0 && (!lx || !cx)) || (ny > 0 && (!ly || !cy)) || !n_out) return -GELIB_HIP_ERR_NULL;
  for (int i = 0; i < len; i++) n_out[i] = 0;
  int count = 0;
  for (int p = 0; p < nx; p++)
    for (int q = 0; q < ny; q++)
      for (int l = std::abs(lx[p] - ly[q]); l <= lx[p] + ly[q]; l++) {
        if (maxl >= 0 && l > maxl) continue;
        if (l >= len) return -GELIB_HIP_ERR_ARG;
        if (n_out[l] == 0) count++;
        n_out[l] += diag ? (int64_t)cx[p] : (int64_t)cx[p] * cy[q];
      }
  return count;
}

int gelib_hip_so3part_cg_fwd(const gelib_part_desc *r, const gelib_part_desc *x, const gelib_part_desc *y, int offs,
                             int accumulate, void *stream) {
  return part_entry(kFwd, false, r, x, y, offs, accumulate, stream);
}
int gelib_hip_so3part_cg_back0(const gelib_part_desc *xg, const gelib_part_desc *g, const gelib_part_desc *y,
                               int offs, int accumulate, void *stream) {
  return part_entry(kBack0, false, g, xg, y, offs, accumulate, stream);
}
int gelib_hip_so3part_cg_back1(const gelib_part_desc *yg, const gelib_part_desc *g, const gelib_part_desc *x,
                               int offs, int accumulate, void *stream) {
  return part_entry(kBack1, false, g, x, yg, offs, accumulate, stream);
}
int gelib_hip_so3part_diagcg_fwd(const gelib_part_desc *r, const gelib_part_desc *x, const gelib_part_desc *y,
                                 int offs, int accumulate, void *stream) {
  return part_entry(kFwd, true, r, x, y, offs, accumulate, stream);
}
int gelib_hip_so3part_diagcg_back0(const gelib_part_desc *xg, const gelib_part_desc *g, const gelib_part_desc *y,
                                   int offs, int accumulate, void *stream) {
  return part_entry(kBack0, true, g, xg, y, offs, accumulate, stream);
}
int gelib_hip_so3part_diagcg_back1(const gelib_part_desc *yg, const gelib_part_desc *g, const gelib_part_desc *x,
                                   int offs, int accumulate, void *stream) {
  return part_entry(kBack1, true, g, x, yg, offs, accumulate, stream);
}

int gelib_hip_so3vec_cg_fwd(int nr, const gelib_part_desc *r, int nx, const gelib_part_desc *x, int ny,
                            const gelib_part_desc *y, int accumulate, void *stream) {
  return vec_fwd_entry(false, nr, r, nx, x, ny, y, accumulate, stream);
}
int gelib_hip_so3vec_cg_bwd(const gelib_part_desc *xg, const gelib_part_desc *yg, int ng, const gelib_part_desc *g,
                            int nx, const gelib_part_desc *x, int ny, const gelib_part_desc *y, int accumulate,
                            void *stream) {
  return vec_bwd_entry(false, xg, yg, ng, g, nx, x, ny, y, accumulate, stream);
}
int gelib_hip_so3vec_diagcg_fwd(int nr, const gelib_part_desc *r, int nx, const gelib_part_desc *x, int ny,
                                const gelib_part_desc *y, int accumulate, void *stream) {
  return vec_fwd_entry(true, nr, r, nx, x, ny, y, accumulate, stream);
}
int gelib_hip_so3vec_diagcg_bwd(const gelib_part_desc *xg, const gelib_part_desc *yg, int ng,
                                const gelib_part_desc *g, int nx, const gelib_part_desc *x, int ny,
                                const gelib_part_desc *y, int accumulate, void *stream) {
  return vec_bwd_entry(true, xg, yg, ng, g, nx, x, ny, y, accumulate, stream);
}

int gelib_hip_so3vec_cg_linear_fwd(int nr, const gelib_part_desc *r, int nx, const gelib_part_desc *x, int ny,
                                   const gelib_part_desc *y, const void *const *w, int accumulate, void *workspace,
                                   uint64_t workspace_bytes, void *stream) {
  return linear_fwd_entry(nr, r, nx, x, ny, y, w, accumulate, workspace, workspace_bytes, stream);
}
int gelib_hip_so3vec_cg_linear_bwd(const gelib_part_desc *xg, const gelib_part_desc *yg, void *const *wg, int ng,
                                   const gelib_part_desc *g, int nx, const gelib_part_desc *x, int ny,
                                   const gelib_part_desc *y, const void *const *w, int accumulate, void *workspace,
                                   uint64_t workspace_bytes, void *stream) {
  return linear_bwd_entry(xg, yg, wg, ng, g, nx, x, ny, y, w, accumulate, workspace, workspace_bytes, stream);
}
uint64_t gelib_hip_so3vec_cg_linear_bwd_workspace_bytes(int ng, const gelib_part_desc *g, int nx, const gelib_part_desc *x,
                                                        int ny, const gelib_part_desc *y, int64_t batch_chunk) {
  LinBwdShape sh;
  if (lin_bwd_shape(ng, g, nx, x, ny, y, nullptr, nullptr, sh)) return 0;
  const long long cb = batch_chunk > 0 ? std::min<long long>(batch_chunk, sh.plan.E[0]) : sh.plan.E[0];
  if (cb <= 0) return 0;
  return (uint64_t)lin_bwd_bytes(sh, cb, nullptr, nullptr, nullptr, nullptr);
}
uint64_t gelib_hip_so3vec_cg_linear_workspace_bytes(int nr, const gelib_part_desc *r, int nx, const gelib_part_desc *x,
                                                    int ny, const gelib_part_desc *y) {
  std::vector<View> R, X, Y;
  if (sort_parts(nr, r, kMaxOutParts, R) || sort_parts(nx, x, kMaxParts, X) || sort_parts(ny, y, kMaxParts, Y)) return 0;
  VecPlan plan;
  if (R.empty() || X.empty() || Y.empty() || build_vec_plan(false, R, X, Y, plan, false)) return 0;
  const std::vector<long long> tau = product_channels(plan, R.size());
  if (R.size() != (size_t)kLinL + 1) return 0;
  long long t5[kLinL + 1];
  for (int l = 0; l <= kLinL; l++) {
    if (R[l].l != l) return 0;
    t5[l] = tau[l];
  }
  long long x_elems = 0;
  for (auto &v : X) x_elems += (long long)(2 * v.l + 1) * v.n;
  return (uint64_t)cg_linear_workspace_bytes(t5, x_elems, plan.E[0] * plan.E[1] * plan.E[2]);
}

int gelib_hip_so3part_spharm(const gelib_part_desc *r, const float *x, const int64_t xdims[5],
                             const int64_t xstrides[5], int accumulate, void *stream) {
  t_last_path = kPathNone;
  View R;
  int rc = check_desc(r, R);
  if (rc) return rc;
  if (!xdims || !xstrides) return GELIB_HIP_ERR_NULL;
  if (xdims[3] != 3 || xdims[4] != R.n) return GELIB_HIP_ERR_ARG;  // (.., 3, n) vectors, one per channel
  long long D[3], xs[5];
  for (int k = 0; k < 3; k++) {
    D[k] = r->dims[k];
    if (xdims[k] != r->dims[k] && xdims[k] != 1) return k == 0 ? GELIB_HIP_ERR_BATCH : GELIB_HIP_ERR_GRID;
    xs[k] = (xdims[k] == r->dims[k] && r->dims[k] > 1) ? xstrides[k] : 0;
  }
  xs[3] = xstrides[3];
  xs[4] = xstrides[4];
  const bool empty = D[0] * D[1] * D[2] == 0 || R.n == 0;
  if (empty) return GELIB_HIP_OK;
  if (!x) return GELIB_HIP_ERR_NULL;
  for (int k = 0; k < 3; k++)
    if (r->dims[k] > 1 && r->strides[k] == 0) return GELIB_HIP_ERR_BROADCAST_DEST;
  if ((rc = check_pointer(r)) || (rc = check_range(x, xdims, xstrides, sizeof(float)))) return rc;
  long long own[3];
  const long long E[3] = {D[0], D[1], D[2]};
  PartDev pr = to_dev(r, E, own);
  t_last_path = kPathGeneric;
  return launch_spharm(pr, x, xs, D, R.l, R.n, accumulate != 0, (hipStream_t)stream);
}

// ---- gather maps -------------------------------------------------------------------------------------------
namespace {

struct GatherMap {  // both directions of a list of (source, target) pairs, compressed by the index that is written
  int n_in, n_out, device;
  int *rows[2], *cols[2];  // [0]: by target (forward), [1]: by source (the inverse map, for the gradient)
};

int upload_compressed(const int32_t *keys, const int32_t *vals, int64_t npairs, int nkeys, int **rows, int **cols) {
  std::vector<int> ptr((size_t)nkeys + 1, 0), out((size_t)std::max<int64_t>(npairs, 1));
  for (int64_t k = 0; k < npairs; k++) ptr[(size_t)keys[k] + 1]++;
  for (int i = 0; i < nkeys; i++) ptr[(size_t)i + 1] += ptr[i];
  std::vector<int> fill(ptr.begin(), ptr.end() - 1);
  for (int64_t k = 0; k < npairs; k++) out[(size_t)fill[keys[k]]++] = vals[k];  // stable: pairs keep their order
  GELIB_HIP_TRY(hipMalloc((void **)rows, ptr.size() * sizeof(int)));
  GELIB_HIP_TRY(hipMalloc((void **)cols, out.size() * sizeof(int)));
  GELIB_HIP_TRY(hipMemcpy(*rows, ptr.data(), ptr.size() * sizeof(int), hipMemcpyHostToDevice));
  GELIB_HIP_TRY(hipMemcpy(*cols, out.data(), out.size() * sizeof(int), hipMemcpyHostToDevice));
  return GELIB_HIP_OK;
}

}  // namespace

int gelib_hip_gather_map_create(const int32_t *sources, const int32_t *targets, int64_t npairs, int n_in, int n_out,
                                void **map) {
  if (!map) return GELIB_HIP_ERR_NULL;
  *map = nullptr;
  if (npairs < 0 || n_in < 0 || n_out < 0 || npairs > 0x7fffffffLL) return GELIB_HIP_ERR_ARG;
  if (npairs > 0 && (!sources || !targets)) return GELIB_HIP_ERR_NULL;
  for (int64_t k = 0; k < npairs; k++)
    if (sources[k] < 0 || sources[k] >= n_in || targets[k] < 0 || targets[k] >= n_out) return GELIB_HIP_ERR_ARG;
  GatherMap *m = new GatherMap();
  m->n_in = n_in;
  m->n_out = n_out;
  m->rows[0] = m->rows[1] = m->cols[0] = m->cols[1] = nullptr;
  hipError_t e = hipGetDevice(&m->device);
  int rc = e == hipSuccess ? GELIB_HIP_OK : record_hip_error(e, "hipGetDevice");
  if (!rc) rc = upload_compressed(targets, sources, npairs, n_out, &m->rows[0], &m->cols[0]);
  if (!rc) rc = upload_compressed(sources, targets, npairs, n_in, &m->rows[1], &m->cols[1]);
  if (rc) {
    gelib_hip_gather_map_destroy(m);
    return rc;
  }
  *map = m;
  return GELIB_HIP_OK;
}

int gelib_hip_gather_map_destroy(void *map) {
  GatherMap *m = (GatherMap *)map;
  if (!m) return GELIB_HIP_OK;
  for (int k = 0; k < 2; k++) {
    if (m->rows[k]) (void)hipFree(m->rows[k]);
    if (m->cols[k]) (void)hipFree(m->cols[k]);
  }
  delete m;
  return GELIB_HIP_OK;
}

int gelib_hip_part_gather(const gelib_part_desc *r, const gelib_part_desc *x, const void *map, int dim, int inverse,
                          int accumulate, void *stream) {
  t_last_path = kPathNone;
  const GatherMap *m = (const GatherMap *)map;
  if (!m) return GELIB_HIP_ERR_NULL;
  View R, X;
  int rc;
  if ((rc = check_desc(r, R)) || (rc = check_desc(x, X))) return rc;
  if (dim < 0 || dim > 2) return GELIB_HIP_ERR_ARG;
  const int dir = inverse ? 1 : 0;
  const int n_from = inverse ? m->n_out : m->n_in, n_to = inverse ? m->n_in : m->n_out;
  for (int k = 0; k < 5; k++) {
    if (k == dim) {
      if (x->dims[k] != n_from || r->dims[k] != n_to) return k == 0 ? GELIB_HIP_ERR_BATCH : GELIB_HIP_ERR_GRID;
    } else if (x->dims[k] != r->dims[k]) {
      return k == 0 ? GELIB_HIP_ERR_BATCH : (k < 3 ? GELIB_HIP_ERR_GRID : GELIB_HIP_ERR_CHANNELS);
    }
  }
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev != m->device) return GELIB_HIP_ERR_DEVICE;
  long long D[5], rs[5], xs[5], total = 1;
  for (int k = 0; k < 5; k++) {
    D[k] = r->dims[k];
    rs[k] = r->strides[k];
    xs[k] = x->strides[k];
    total *= D[k];
    if (r->dims[k] > 1 && r->strides[k] == 0) return GELIB_HIP_ERR_BROADCAST_DEST;
  }
  if (total == 0) return GELIB_HIP_OK;
  if (!r->ptr || (!x->ptr && n_from > 0)) return GELIB_HIP_ERR_NULL;
  if ((rc = check_pointer(r)) || (rc = check_pointer(x))) return rc;
  t_last_path = kPathGeneric;
  return launch_gather((float2 *)r->ptr, (const float2 *)x->ptr, rs, xs, D, dim, m->rows[dir], m->cols[dir],
                       accumulate != 0, (hipStream_t)stream);
}

// ---- channel mixing (the linear layer that consumes a product) ------------------------------------------------------
namespace {
// argument checks shared by the two forms of the product; 0 = go on, -1 = nothing to do, else a status
int mix_check(void *r, const void *x, const void *w, int64_t rows, int n_in, int n_out, int64_t r_row_stride,
              int64_t x_row_stride, int adjoint) {
  if (rows < 0 || n_in < 0 || n_out < 0 || r_row_stride < n_out || x_row_stride < n_in) return GELIB_HIP_ERR_ARG;
  if (rows == 0 || n_out == 0) return -1;
  if (!r || (n_in > 0 && (!x || !w))) return GELIB_HIP_ERR_NULL;
  if (n_in == 0 || (n_in & 1) || (x_row_stride & 1) || ((uintptr_t)x & 15) || rows > (1LL << 38))
    return GELIB_HIP_ERR_ARG;
  const int64_t rd[5] = {rows, 1, 1, 1, n_out}, rst[5] = {r_row_stride, 0, 0, 0, 1};
  const int64_t xd[5] = {rows, 1, 1, 1, n_in}, xst[5] = {x_row_stride, 0, 0, 0, 1};
  const int64_t wd[5] = {adjoint ? n_out : n_in, 1, 1, 1, adjoint ? n_in : n_out};
  const int64_t wst[5] = {wd[4], 0, 0, 0, 1};
  int rc;
  if ((rc = check_range(r, rd, rst, 2 * sizeof(float))) || (rc = check_range(x, xd, xst, 2 * sizeof(float))) ||
      (rc = check_range(w, wd, wst, 2 * sizeof(float))))
    return rc;
  return GELIB_HIP_OK;
}
}  // namespace

int gelib_hip_part_mix_channels(void *r, const void *x, const void *w, int64_t rows, int n_in, int n_out,
                                int64_t r_row_stride, int64_t x_row_stride, int adjoint, void *workspace,
                                uint64_t workspace_bytes, void *stream) {
  t_last_path = kPathNone;
  int rc = mix_check(r, x, w, rows, n_in, n_out, r_row_stride, x_row_stride, adjoint);
  if (rc) return rc < 0 ? GELIB_HIP_OK : rc;
  const int64_t sd[5] = {(int64_t)workspace_bytes, 1, 1, 1, 1}, sst[5] = {1, 0, 0, 0, 0};
  if (workspace && workspace_bytes && (rc = check_range(workspace, sd, sst, 1))) return rc;
  t_last_path = kPathGeneric;
  rc = launch_mix((float2 *)r, (const float2 *)x, (const float2 *)w, rows, n_in, n_out, x_row_stride, r_row_stride,
                  adjoint != 0, (float *)workspace, (size_t)workspace_bytes, (hipStream_t)stream);
  return rc == 11 ? GELIB_HIP_ERR_ARG : rc;
}

int gelib_hip_part_mix_channels_static(void *r, const void *x, const void *w, int64_t rows, int n_in, int n_out,
                                       int64_t r_row_stride, int64_t x_row_stride, int adjoint, void *stream) {
  t_last_path = kPathNone;
  int rc = mix_check(r, x, w, rows, n_in, n_out, r_row_stride, x_row_stride, adjoint);
  if (rc) return rc < 0 ? GELIB_HIP_OK : rc;
  t_last_path = kPathGeneric;
  rc = launch_mix_static((float2 *)r, (const float2 *)x, (const float2 *)w, rows, n_in, n_out, x_row_stride,
                         r_row_stride, adjoint != 0, (hipStream_t)stream);
  return rc == 11 ? GELIB_HIP_ERR_ARG : rc;
}

int gelib_hip_part_mix_channels_wgrad(void *wg, const void *x, const void *g, int64_t rows, int n_in, int n_out,
                                      int64_t x_row_stride, int64_t g_row_stride, void *workspace,
                                      uint64_t workspace_bytes, void *stream) {
  t_last_path = kPathNone;
  if (rows < 0 || n_in < 0 || n_out < 0 || x_row_stride < n_in || g_row_stride < n_out) return GELIB_HIP_ERR_ARG;
  if (n_in == 0 || n_out == 0) return GELIB_HIP_OK;
  if (!wg || (rows > 0 && (!x || !g))) return GELIB_HIP_ERR_NULL;
  if ((n_in & 1) || (x_row_stride & 1) || ((uintptr_t)x & 15) || rows > (1LL << 38)) return GELIB_HIP_ERR_ARG;
  const int64_t xd[5] = {rows, 1, 1, 1, n_in}, xst[5] = {x_row_stride, 0, 0, 0, 1};
  const int64_t gd[5] = {rows, 1, 1, 1, n_out}, gst[5] = {g_row_stride, 0, 0, 0, 1};
  const int64_t wd[5] = {n_in, 1, 1, 1, n_out}, wst[5] = {n_out, 0, 0, 0, 1};
  int rc;
  if ((rc = check_range(wg, wd, wst, 2 * sizeof(float))) || (rc = check_range(x, xd, xst, 2 * sizeof(float))) ||
      (rc = check_range(g, gd, gst, 2 * sizeof(float))))
    return rc;
  const int64_t sd[5] = {(int64_t)workspace_bytes, 1, 1, 1, 1}, sst[5] = {1, 0, 0, 0, 0};
  if (workspace && workspace_bytes && (rc = check_range(workspace, sd, sst, 1))) return rc;
  t_last_path = kPathGeneric;
  rc = launch_mix_wgrad((float2 *)wg, (const float2 *)x, (const float2 *)g, rows, n_in, n_out, x_row_stride,
                        g_row_stride, (float *)workspace, (size_t)workspace_bytes, (hipStream_t)stream);
  return rc == 11 ? GELIB_HIP_ERR_ARG : rc;
}

uint64_t gelib_hip_part_mix_workspace_bytes(int kind, int64_t rows, int n_in, int n_out) {
  if (rows <= 0 || n_in <= 0 || n_out <= 0) return 0;
  if (kind == 0) return mix_workspace_bytes(n_in, n_out);
  if (kind == 1) return mix_wgrad_workspace_bytes(rows, n_in, n_out);
  return 0;
}

int gelib_hip_set_stream_workspace(void *stream, void *ptr, uint64_t bytes) {
  int dev = 0;
  GELIB_HIP_TRY(hipGetDevice(&dev));
  if (ptr && bytes) {
    if ((uintptr_t)ptr & 255) return GELIB_HIP_ERR_WORKSPACE;
    const int64_t sd[5] = {(int64_t)bytes, 1, 1, 1, 1}, sst[5] = {1, 0, 0, 0, 0};
    int rc = check_range(ptr, sd, sst, 1);
    if (rc) return rc;
  }
  // both scratch users finish putting their kernels on the stream before the buffer changes under them
  std::lock_guard<std::mutex> l0(stream_scratch_mutex(0));
  std::lock_guard<std::mutex> l1(stream_scratch_mutex(1));
  std::lock_guard<std::mutex> lock(g_lent_mutex);
  if (ptr && bytes) {
    ScratchBuf b;
    b.ptr = (char *)ptr;
    b.bytes = (size_t)bytes;
    g_lent[{dev, (hipStream_t)stream}] = b;
  } else {
    g_lent.erase({dev, (hipStream_t)stream});
  }
  return GELIB_HIP_OK;
}

int gelib_hip_malloc(void **ptr, uint64_t bytes) {
  if (!ptr) return GELIB_HIP_ERR_NULL;
  *ptr = nullptr;
  if (bytes == 0) return GELIB_HIP_OK;
  GELIB_HIP_TRY(hipMalloc(ptr, bytes));
  return GELIB_HIP_OK;
}
int gelib_hip_free(void *ptr) {
  if (ptr) forget_ranges(ptr);  // the pointer check must not pass views into memory that is gone
  if (ptr) GELIB_HIP_TRY(hipFree(ptr));
  return GELIB_HIP_OK;
}
int gelib_hip_memcpy(void *dst, const void *src, uint64_t bytes, int kind) {
  if (bytes == 0) return GELIB_HIP_OK;
  if (!dst || !src) return GELIB_HIP_ERR_NULL;
  const hipMemcpyKind k = kind == 0 ? hipMemcpyHostToDevice : (kind == 1 ? hipMemcpyDeviceToHost : hipMemcpyDeviceToDevice);
  if (kind < 0 || kind > 2) return GELIB_HIP_ERR_ARG;
  GELIB_HIP_TRY(hipMemcpy(dst, src, bytes, k));
  return GELIB_HIP_OK;
}
int gelib_hip_memset(void *ptr, int value, uint64_t bytes) {
  if (bytes == 0) return GELIB_HIP_OK;
  if (!ptr) return GELIB_HIP_ERR_NULL;
  GELIB_HIP_TRY(hipMemset(ptr, value, bytes));
  return GELIB_HIP_OK;
}
int gelib_hip_synchronize(void) {
  GELIB_HIP_TRY(hipDeviceSynchronize());
  return GELIB_HIP_OK;
}

int gelib_hip_set_option(const char *name, int value) {
  if (!name) return GELIB_HIP_ERR_NULL;
  if (!std::strcmp(name, "force_generic")) {
    g_force_generic = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "pairwise_bwd")) {  // 0 never, 1 for operand l above 7, 2 wherever every pair qualifies
    g_pairwise = value;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "check_pointers")) {
    g_check_pointers = value;
    forget_ranges(nullptr);
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "bcast_scratch_kb")) {  // KiB the temporary of a broadcast gradient destination may take
    g_bcast_scratch_kb = value > 0 ? value : 64 * 1024;
    return GELIB_HIP_OK;
  }
  if (!std::strcmp(name, "bcast_reduce")) {  // 0: sum a broadcast destination inside the shape-agnostic kernels
    g_bcast_reduce = value;
    return GELIB_HIP_OK;
  }
  if (!std::strncmp(name, "staged_", 7)) return staged_set_option(name, value);
  if (!std::strncmp(name, "diag6", 5)) return diag6_set_option(name, value);
  if (!std::strncmp(name, "onepair_mfma", 12)) return onepair_mfma_set_option(name, value);
  if (!std::strncmp(name, "onepair", 7)) return onepair_set_option(name, value);
  if (!std::strncmp(name, "mix_", 4)) return mix_set_option(name, value);
  return unrolled_set_option(name, value);
}

int gelib_hip_last_path(void) { return t_last_path; }

}  // extern "C"
