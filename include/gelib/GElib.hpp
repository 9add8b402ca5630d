// C++ host-side mirror of GElib's interface for the Clebsch-Gordan product path, over libgelib_hip.so.
//
// Same names, namespaces and argument orders as the reference, so code written against GElib's SO3part /
// SO3vec / CGproduct API for this path compiles against this header:
//   GElib::SO3group, SO3type          SO3/SO3group.hpp:21-55, SO3/SO3type.hpp:21-47, core/Gtype.hpp:115-138
//   GElib::SO3CGbank, SO3_CGbank      SO3/SO3CGbank.hpp:26-95, include/GElib_base.cpp:20
//   GElib::SO3part<float>             SO3/SO3part.hpp:42-335 (constructors, getl/getn/getb, CG kernels' seams)
//   GElib::SO3vec<float>              SO3/SO3vec.hpp:26-65, core/Gvec.hpp:25-389
//   CGproduct / DiagCGproduct         core/CGproduct.hpp:32-41,120-124, core/DiagCGproduct.hpp:32-41
//   Gpart_add_CGproduct[_back0/1]     core/CGproduct.hpp:44-104 (dest, then the others, then offs)
//   Gpart_add_DiagCGproduct[_back0/1] core/DiagCGproduct.hpp:44-105
// Device convention as in the reference: dev 0 = host memory, dev 1 = GPU0 (SO3/SO3CGbank.hpp:37-49).
// The arithmetic of dev==1 parts runs in the HIP kernels behind the C ABI; parts on dev 0 can be created, filled
// and transported, but products of host parts are not part of this build and throw.
// Where the reference prints "... skipped ..." and returns (GELIB_SKIP, include/GElib_base.hpp:36) this mirror
// throws std::runtime_error with the same text, so a shape mistake cannot pass silently.
#pragma once

#include <cmath>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <sstream>
#include <stdexcept>
#include <unordered_map>

#include "cnine_min.hpp"

#define _GELIB_VERSION "gelib-mi355x-cg 0.1"

#define GELIB_ASSRT(condition) \
  if (!(condition))            \
    throw std::runtime_error("GElib error in " + std::string(__PRETTY_FUNCTION__) + " : failed assertion " + #condition + ".");
#define GELIB_ERROR(msg) throw std::runtime_error("GElib error in " + std::string(__PRETTY_FUNCTION__) + " : " + msg + ".");
#define GELIB_SKIP(msg) throw std::runtime_error("Function " + std::string(__func__) + " skipped: " + msg + ".");

namespace GElib {
inline void gelib_check(const int rc);
}

namespace cnine {

// A list of (source, target) pairs: slice `target` of the result collects slice `source` of the argument
// (the class python/bindings/gather_map_py.cpp:15-29 binds; its definition is in cnine, outside the reference tree).
// Pairs keep their order within one target, which fixes the order of the float sums.  The device form is made on
// first use, on the GPU that is current then, and released with the last copy of the map.
class GatherMapB {
 public:
  int n_in = 0, n_out = 0;
  std::vector<int> sources, targets;
  bool inverted = false;

  GatherMapB() {}
  // n_in / n_out default to the largest index + 1
  GatherMapB(const std::vector<int> &_sources, const std::vector<int> &_targets, const int _n_in = -1, const int _n_out = -1)
      : sources(_sources), targets(_targets) {
    if (sources.size() != targets.size()) throw std::invalid_argument("GatherMapB: as many sources as targets are needed.");
    int ms = -1, mt = -1;
    for (size_t i = 0; i < sources.size(); i++) ms = std::max(ms, sources[i]), mt = std::max(mt, targets[i]);
    n_in = _n_in < 0 ? ms + 1 : _n_in;
    n_out = _n_out < 0 ? mt + 1 : _n_out;
    for (size_t i = 0; i < sources.size(); i++)
      if (sources[i] < 0 || sources[i] >= n_in || targets[i] < 0 || targets[i] >= n_out)
        throw std::out_of_range("GatherMapB: index outside [0, n_in) x [0, n_out).");
  }
  // rows of M are (source, target)
  GatherMapB(const TensorView<int> &M, const int _n_in, const int _n_out) : n_in(_n_in), n_out(_n_out) {
    if (M.ndims() != 2 || M.dim(1) != 2) throw std::invalid_argument("GatherMapB: the matrix must be k x 2.");
    if (M.get_dev() != 0) throw std::invalid_argument("GatherMapB: the matrix must be in host memory.");
    for (int i = 0; i < M.dim(0); i++) {
      sources.push_back(M.arr[i * M.strides[0]]);
      targets.push_back(M.arr[i * M.strides[0] + M.strides[1]]);
    }
    *this = GatherMapB(sources, targets, n_in, n_out);
  }
  // every (source, target) pair independently with probability p
  static GatherMapB random(const int n_in, const int n_out, const float p, const unsigned seed = 0) {
    std::vector<int> s, t;
    unsigned long long state = 0x9E3779B97F4A7C15ull ^ seed;
    for (int j = 0; j < n_out; j++)
      for (int i = 0; i < n_in; i++) {
        state = state * 6364136223846793005ull + 1442695040888963407ull;
        if ((double)(state >> 11) / 9007199254740992.0 < p) s.push_back(i), t.push_back(j);
      }
    return GatherMapB(s, t, n_in, n_out);
  }

  GatherMapB inv() const {  // same pairs read backwards (core/Gpart.hpp:561)
    GatherMapB R(*this);
    R.inverted = !inverted;
    return R;
  }
  int d_in() const { return inverted ? n_out : n_in; }
  int d_out() const { return inverted ? n_in : n_out; }
  size_t size() const { return sources.size(); }

  void *device_handle() const {
    if (!handle) {
      void *h = nullptr;
      GElib::gelib_check(gelib_hip_gather_map_create(sources.data(), targets.data(), (int64_t)sources.size(), n_in, n_out, &h));
      handle = std::shared_ptr<void>(h, [](void *q) { gelib_hip_gather_map_destroy(q); });
    }
    return handle.get();
  }

  std::string str(const std::string indent = "") const {
    std::ostringstream oss;
    for (int t = 0; t < d_out(); t++) {
      oss << indent << t << "<-(";
      bool first = true;
      for (size_t k = 0; k < size(); k++)
        if ((inverted ? sources[k] : targets[k]) == t) {
          oss << (first ? "" : ",") << (inverted ? targets[k] : sources[k]);
          first = false;
        }
      oss << ")\n";
    }
    return oss.str();
  }
  std::string repr() const {
    std::ostringstream oss;
    oss << "<cnine::GatherMapB n_in=" << d_in() << " n_out=" << d_out() << " pairs=" << size() << ">";
    return oss.str();
  }

 private:
  mutable std::shared_ptr<void> handle;
};

}  // namespace cnine

namespace GElib {

class GtypeBase {};
class GpartBase {};
class GvecBase {};

// HIP stream the products are queued on (per thread; nullptr = the default stream).  The PyTorch binding sets it
// to torch's current stream before every call, where the reference creates a private stream per call
// (CUDA_STREAM, SO3/SO3part.hpp:260).
inline void *&gelib_stream() {
  thread_local void *s = nullptr;
  return s;
}

// 1 = the reference's "+=" into the destination (default); 0 = overwrite, for callers that hand in uninitialised
// outputs instead of zero-filled ones (SO3vec level only).
inline int &accumulate_mode() {
  thread_local int a = 1;
  return a;
}

inline void gelib_check(const int rc) {
  if (rc == 0) return;
  std::string msg = gelib_hip_strerror(rc);
  if (rc == GELIB_HIP_ERR_RUNTIME) msg += std::string(": ") + gelib_hip_last_runtime_error();
  throw std::runtime_error("GElib error: " + msg + ".");
}

// ---- SO3group -----------------------------------------------------------------------------------------------

class SO3type;

class SO3group {
 public:
  typedef int IRREP_IX;
  typedef int GINDEX;
  typedef SO3type GTYPE;

  static int CGmultiplicity(const int l1, const int l2, const int l) {
    return (l >= std::abs(l1 - l2) && l <= l1 + l2) ? 1 : 0;
  }
  static void for_each_CGcomponent(const int l1, const int l2, const std::function<void(const int l, const int m)> &lambda) {
    for (int l = std::abs(l1 - l2); l <= l1 + l2; l++) lambda(l, 1);
  }
  static int CG_sign_rule(const int l1, const int l2, const int l) { return 1 - 2 * ((l1 + l2 - l) % 2); }
};

// ---- SO3type ------------------------------------------------------------------------------------------------

class SO3type : public GtypeBase {
 public:
  typedef int IRREP_IX;
  typedef SO3group Group;
  static constexpr int null_ix = -1;

  mutable std::map<int, int> parts;

  SO3type() {}
  SO3type(const std::map<int, int> &_parts) : parts(_parts) {}
  SO3type(const std::initializer_list<std::pair<int, int>> &list) {
    for (auto p : list) parts[p.first] = p.second;
  }
  SO3type(const std::vector<int> &v) {
    int l = 0;
    for (auto &p : v) parts[l++] = p;
  }

  int size() const { return (int)parts.size(); }
  int highest() const { return parts.crbegin()->first; }
  int &operator[](const int ix) { return parts[ix]; }
  int operator()(const int ix) const {
    auto it = parts.find(ix);
    return it == parts.end() ? 0 : it->second;
  }
  void set(const int ix, const int n) { parts[ix] = n; }
  bool operator==(const SO3type &y) const { return parts == y.parts; }

  // Type of the product: channels of part l = sum over the pairs (l1, l2) with |l1 - l2| <= l <= l1 + l2 of n1 n2
  // (Diag: n1); a limit >= 0 keeps the parts up to it (core/Gtype.hpp:115-138).
  SO3type CGproduct(const SO3type &y, const int limit = null_ix) const { return product_type(y, limit, false); }
  SO3type DiagCGproduct(const SO3type &y, const int limit = null_ix) const { return product_type(y, limit, true); }

 private:
  SO3type product_type(const SO3type &y, const int limit, const bool diag) const {
    SO3type R;
    for (const auto &[l1, n1] : parts)
      for (const auto &[l2, n2] : y.parts) {
        const int top = limit == null_ix ? l1 + l2 : std::min(l1 + l2, limit);
        for (int l = std::abs(l1 - l2); l <= top; l++) R.parts[l] += diag ? n1 : n1 * n2;
      }
    return R;
  }

 public:
  std::string str(const std::string indent = "") const {
    std::ostringstream oss;
    oss << indent << "(";
    bool first = true;
    for (auto &p : parts) {
      oss << (first ? "" : ",") << p.first << ":" << p.second;
      first = false;
    }
    oss << ")";
    return oss.str();
  }
  std::string repr() const { return "<SO3type " + str() + ">"; }
};

inline SO3type CGproduct(const SO3type &x, const SO3type &y, const int maxl = -1) { return x.CGproduct(y, maxl); }
inline SO3type DiagCGproduct(const SO3type &x, const SO3type &y, const int maxl = -1) { return x.DiagCGproduct(y, maxl); }

// ---- SO3CGbank ----------------------------------------------------------------------------------------------

struct SO3CGindex {
  int l1, l2, l;
  bool operator==(const SO3CGindex &x) const { return l1 == x.l1 && l2 == x.l2 && l == x.l; }
};
struct SO3CGindexHash {
  size_t operator()(const SO3CGindex &ix) const { return ((size_t)ix.l1 << 20) ^ ((size_t)ix.l2 << 10) ^ (size_t)ix.l; }
};

// Host-side coefficient bank (row-major (2l1+1)x(2l2+1) float tables, cached; guarded by a mutex).  The GPU
// kernels keep their own device-side copies inside the library.
class SO3CGbank {
 public:
  typedef cnine::TensorView<float> FTENSOR;

  template <typename TYPE>
  cnine::TensorView<TYPE> &get(const int l1, const int l2, const int l, const int dev = 0) {
    static_assert(std::is_same<TYPE, float>::value, "Currenly only single precision CG matrices supported.");
    if (dev != 0) GELIB_ERROR("the device copies of the CG matrices live inside libgelib_hip; ask for dev=0");
    if (l < std::abs(l1 - l2) || l > l1 + l2) GELIB_ERROR("|l1-l_2| <= l <= l1+l2 not satisfied");
    std::lock_guard<std::mutex> lock(mx);
    SO3CGindex ix{l1, l2, l};
    auto it = coeffsf.find(ix);
    if (it != coeffsf.end()) return it->second;
    FTENSOR R(cnine::Gdims({2 * l1 + 1, 2 * l2 + 1}), 0, 0);
    gelib_check(gelib_hip_cg_matrix(l1, l2, l, R.arr));
    return coeffsf.emplace(ix, R).first->second;
  }

 private:
  std::mutex mx;
  std::unordered_map<SO3CGindex, FTENSOR, SO3CGindexHash> coeffsf;
};

inline SO3CGbank &SO3_CGbank_instance() {
  static SO3CGbank bank;
  return bank;
}
#define SO3_CGbank (::GElib::SO3_CGbank_instance())

// ---- SO3part ------------------------------------------------------------------------------------------------

template <typename TYPE>
class SO3part : public cnine::BatchedTensor<std::complex<TYPE>>, public GpartBase {
 public:
  typedef cnine::BatchedTensor<std::complex<TYPE>> BASE;
  typedef cnine::TensorView<std::complex<TYPE>> TENSOR;
  typedef cnine::TensorView<TYPE> RTENSOR;
  typedef cnine::Gdims Gdims;
  typedef SO3group GROUP;
  typedef int IRREP_IX;
  typedef SO3type GTYPE;
  static constexpr int null_ix = -1;

  using BASE::arr;
  using BASE::dev;
  using BASE::dims;
  using BASE::getb;
  using BASE::ndims;
  using BASE::strides;

  SO3part() {}
  SO3part(const int _b, const int _l, const int _nc, const int _fcode = 0, const int _dev = 0)
      : BASE(Gdims({_b, 2 * _l + 1, _nc}), _fcode, _dev) {}
  SO3part(const int _b, const Gdims &_gdims, const int _l, const int _nc, const int _fcode = 0, const int _dev = 0)
      : BASE(Gdims(_b, _gdims, {2 * _l + 1, _nc}), _fcode, _dev) {}
  SO3part(const int _l, const int _b, const Gdims &_gdims, const int _nc, const int _fcode = 0, const int _dev = 0)
      : BASE(Gdims(_b, _gdims, {2 * _l + 1, _nc}), _fcode, _dev) {}

  // conversion from a tensor view (aliases the memory)
  SO3part(const TENSOR &x) : BASE(x) {
    GELIB_ASSRT(ndims() >= 3);
    GELIB_ASSRT(dims(-2) % 2 == 1);
  }
  // transport
  SO3part(const SO3part &x, const int _dev) : SO3part(TENSOR(x, _dev)) {}

  SO3part zeros_like() const { return SO3part(TENSOR(dims, 0, dev)); }

  int get_ix() const { return (dims(-2) - 1) / 2; }
  int getl() const { return (dims(-2) - 1) / 2; }
  int getn() const { return dims.last(); }
  int get_dev() const { return dev; }
  Gdims get_gdims() const { return dims.chunk(1, (int)dims.size() - 3); }
  int dominant_batch(const SO3part &y) const { return std::max(getb(), y.getb()); }
  Gdims dominant_gdims(const SO3part &y) const { return ndims() > 3 ? get_gdims() : y.get_gdims(); }

  RTENSOR get_CGmatrix(const SO3part &x, const SO3part &y) { return SO3_CGbank.template get<TYPE>(x.getl(), y.getl(), getl()); }

  // 5-D descriptor (batch, grid0, grid1, 2l+1, n).  More than two grid dimensions are fused into one when their
  // strides nest (core/Gpart.hpp:450-469).
  gelib_part_desc descriptor() const {
    const int d = ndims();
    GELIB_ASSRT(d >= 3);
    gelib_part_desc D;
    D.ptr = (void *)arr;
    long long gd[2] = {1, 1}, gs[2] = {0, 0};
    const int ng = d - 3;
    if (ng == 1) {
      gd[0] = dims[1];
      gs[0] = (long long)strides[1];
    } else if (ng == 2) {
      gd[0] = dims[1];
      gs[0] = (long long)strides[1];
      gd[1] = dims[2];
      gs[1] = (long long)strides[2];
    } else if (ng > 2) {
      long long tot = 1;
      for (int i = 1; i <= ng; i++) tot *= dims[i];
      for (int i = 1; i < ng; i++)
        if (strides[i] != (size_t)dims[i + 1] * strides[i + 1])
          GELIB_ERROR("the grid dimensions of an SO3part with more than two of them must be fusible");
      gd[0] = tot;
      gs[0] = (long long)strides[ng];
    }
    D.dims[0] = dims[0];
    D.strides[0] = (long long)strides[0];
    D.dims[1] = gd[0];
    D.strides[1] = gs[0];
    D.dims[2] = gd[1];
    D.strides[2] = gs[1];
    D.dims[3] = dims[d - 2];
    D.strides[3] = (long long)strides[d - 2];
    D.dims[4] = dims[d - 1];
    D.strides[4] = (long long)strides[d - 1];
    return D;
  }

  // ---- device seams (SO3/SO3part.hpp:259-269, 324-334): destination first, as in the reference ----
  static void add_CGproduct_dev(const SO3part &r, SO3part x, SO3part y, const int offs = 0) {
    auto R = r.descriptor(), X = x.descriptor(), Y = y.descriptor();
    gelib_check(gelib_hip_so3part_cg_fwd(&R, &X, &Y, offs, 1, gelib_stream()));
  }
  static void add_CGproduct_back0_dev(const SO3part &xg, SO3part g, SO3part y, const int offs = 0) {
    auto XG = xg.descriptor(), G = g.descriptor(), Y = y.descriptor();
    gelib_check(gelib_hip_so3part_cg_back0(&XG, &G, &Y, offs, 1, gelib_stream()));
  }
  static void add_CGproduct_back1_dev(const SO3part &yg, SO3part g, SO3part x, const int offs = 0) {
    auto YG = yg.descriptor(), G = g.descriptor(), X = x.descriptor();
    gelib_check(gelib_hip_so3part_cg_back1(&YG, &G, &X, offs, 1, gelib_stream()));
  }
  static void add_DiagCGproduct_dev(const SO3part &r, SO3part x, SO3part y, const int offs = 0) {
    auto R = r.descriptor(), X = x.descriptor(), Y = y.descriptor();
    gelib_check(gelib_hip_so3part_diagcg_fwd(&R, &X, &Y, offs, 1, gelib_stream()));
  }
  static void add_DiagCGproduct_back0_dev(const SO3part &xg, SO3part g, SO3part y, const int offs = 0) {
    auto XG = xg.descriptor(), G = g.descriptor(), Y = y.descriptor();
    gelib_check(gelib_hip_so3part_diagcg_back0(&XG, &G, &Y, offs, 1, gelib_stream()));
  }
  static void add_DiagCGproduct_back1_dev(const SO3part &yg, SO3part g, SO3part x, const int offs = 0) {
    auto YG = yg.descriptor(), G = g.descriptor(), X = x.descriptor();
    gelib_check(gelib_hip_so3part_diagcg_back1(&YG, &G, &X, offs, 1, gelib_stream()));
  }

  // ---- spherical harmonics (SO3/SO3part.hpp:340-403): x is (.., 3, n) real, leading dims as this part's or 1 ----
  void add_spharm(const cnine::TensorView<float> &x) const {
    GELIB_ASSRT(x.get_dev() == dev);
    if (dev != 1) GELIB_ERROR("SO3part::add_spharm: the operands must be on GPU");
    const int d = ndims(), xd = x.ndims();
    if (xd < 2) GELIB_ERROR("x must be at least 2D.");
    if (x.dim(xd - 2) != 3) GELIB_ERROR("dim(-2) of x must be 3.");
    gelib_part_desc R = descriptor();
    // x without leading dimensions is shared by every cell (cuda/SPharm.cu:101-107)
    int64_t xdims[5] = {1, 1, 1, 3, x.dim(xd - 1)};
    int64_t xstr[5] = {0, 0, 0, (int64_t)x.strides[xd - 2], (int64_t)x.strides[xd - 1]};
    if (xd > 2) {
      if (xd != d) GELIB_ERROR("x must have as many leading dimensions as the part.");
      xdims[0] = x.dim(0);
      xstr[0] = (int64_t)x.strides[0];
      const int ng = xd - 3;
      if (ng == 1 || ng == 2) {
        for (int k = 0; k < ng; k++) xdims[1 + k] = x.dim(1 + k), xstr[1 + k] = (int64_t)x.strides[1 + k];
      } else if (ng > 2) {  // fused like the part's own grid dimensions
        int64_t tot = 1;
        for (int k = 1; k <= ng; k++) tot *= x.dim(k);
        for (int k = 1; k < ng; k++)
          if (x.strides[k] != (size_t)x.dim(k + 1) * x.strides[k + 1])
            GELIB_ERROR("the grid dimensions of x must be fusible when there are more than two of them");
        xdims[1] = tot;
        xstr[1] = (int64_t)x.strides[ng];
      }
    }
    gelib_check(gelib_hip_so3part_spharm(&R, x.arr, xdims, xstr, 1, gelib_stream()));
  }

  // ---- sums of slices along grid dimension d (core/Gpart.hpp:556-562) ----
  void add_gather(const SO3part &x, const cnine::GatherMapB &gmap, const int d = 0) const {
    GELIB_ASSRT(x.dev == dev);
    if (dev != 1) GELIB_ERROR("SO3part::add_gather: the operands must be on GPU");
    GELIB_ASSRT(ndims() <= 5 && x.ndims() == ndims());
    GELIB_ASSRT(d >= 0 && d < ndims() - 3);
    GELIB_ASSRT(gmap.d_in() == x.dims[d + 1]);
    GELIB_ASSRT(gmap.d_out() == dims[d + 1]);
    auto R = descriptor(), X = x.descriptor();
    gelib_check(gelib_hip_part_gather(&R, &X, gmap.device_handle(), d + 1, gmap.inverted ? 1 : 0, 1, gelib_stream()));
  }
  void add_gather_back(const SO3part &r, const cnine::GatherMapB &gmap, const int d = 0) const {
    gmap.device_handle();  // made on the caller's map, so the reversed copy below shares it instead of uploading,
                           // using and freeing a device copy of its own on every call
    add_gather(r, gmap.inv(), d);
  }

  std::string classname() const { return "GElib::SO3part"; }
  std::string repr() const {
    std::ostringstream oss;
    oss << "<GElib::SO3part l=" << getl() << " n=" << getn() << " b=" << getb() << " dev=" << dev << ">";
    return oss.str();
  }
  std::string str(const std::string indent = "") const { return indent + repr(); }
};

// ---- part-level dispatchers (core/CGproduct.hpp:44-104, core/DiagCGproduct.hpp:44-105) -----------------------

namespace detail {
template <typename GPART>
inline void check_devices(const GPART &r, const GPART &x, const GPART &y) {
  GELIB_ASSRT(x.get_dev() == r.get_dev());
  GELIB_ASSRT(y.get_dev() == r.get_dev());
  if (r.get_dev() != 1) GELIB_ERROR("SO3part must be on GPU: products of host parts are not part of this build");
}
inline void skip_on(const int rc) {
  if (rc == GELIB_HIP_ERR_BATCH) GELIB_SKIP("batch dimensions cannot be reconciled");
  if (rc == GELIB_HIP_ERR_GRID) GELIB_SKIP("grid dimensions cannot be reconciled");
  gelib_check(rc);
}
}  // namespace detail

#define GELIB_PART_DISPATCH(NAME, ENTRY)                                                          \
  template <typename GPART>                                                                       \
  void NAME(GPART dest, GPART a, GPART b, const int offs = 0) {                                   \
    detail::check_devices(dest, a, b);                                                            \
    auto D = dest.descriptor(), A = a.descriptor(), B = b.descriptor();                           \
    detail::skip_on(ENTRY(&D, &A, &B, offs, 1, gelib_stream()));                                         \
  }
GELIB_PART_DISPATCH(Gpart_add_CGproduct, gelib_hip_so3part_cg_fwd)              // (r, x, y, offs)
GELIB_PART_DISPATCH(Gpart_add_CGproduct_back0, gelib_hip_so3part_cg_back0)      // (xg, g, y, offs)
GELIB_PART_DISPATCH(Gpart_add_CGproduct_back1, gelib_hip_so3part_cg_back1)      // (yg, g, x, offs)
GELIB_PART_DISPATCH(Gpart_add_DiagCGproduct, gelib_hip_so3part_diagcg_fwd)
GELIB_PART_DISPATCH(Gpart_add_DiagCGproduct_back0, gelib_hip_so3part_diagcg_back0)
GELIB_PART_DISPATCH(Gpart_add_DiagCGproduct_back1, gelib_hip_so3part_diagcg_back1)
#undef GELIB_PART_DISPATCH

template <typename GPART>
typename std::enable_if<std::is_base_of<GpartBase, GPART>::value, GPART>::type CGproduct(const GPART &x, const GPART &y,
                                                                                         const typename GPART::IRREP_IX &ix) {
  int m = GPART::GROUP::CGmultiplicity(x.get_ix(), y.get_ix(), ix);
  GELIB_ASSRT(m > 0);
  GPART R(ix, x.dominant_batch(y), x.dominant_gdims(y), x.getn() * y.getn(), 0, x.dev);
  Gpart_add_CGproduct(R, x, y);
  return R;
}

template <typename GPART>
typename std::enable_if<std::is_base_of<GpartBase, GPART>::value, GPART>::type DiagCGproduct(
    const GPART &x, const GPART &y, const typename GPART::IRREP_IX &ix) {
  int m = GPART::GROUP::CGmultiplicity(x.get_ix(), y.get_ix(), ix);
  GELIB_ASSRT(m > 0);
  GELIB_ASSRT(x.getn() == y.getn());
  GPART R(ix, x.dominant_batch(y), x.dominant_gdims(y), x.getn(), 0, x.dev);
  Gpart_add_DiagCGproduct(R, x, y);
  return R;
}

// ---- SO3vec ---------------------------------------------------------------------------------------------------

template <typename TYPE>
class SO3vec : public GvecBase {
 public:
  typedef SO3part<TYPE> GPART;
  typedef cnine::Gdims Gdims;
  typedef SO3type GTYPE;
  typedef int IRREP_IX;

  int _nbatch = 0;
  Gdims _gdims;
  int dev = 0;
  mutable std::map<int, GPART> parts;

  SO3vec() {}
  SO3vec(const int __nbatch, const Gdims &__gdims, const int _dev = 0) : _nbatch(__nbatch), _gdims(__gdims), dev(_dev) {}
  SO3vec(const int __nbatch, const Gdims &__gdims, const SO3type &tau, const int fcode = 0, const int _dev = 0)
      : SO3vec(__nbatch, __gdims, _dev) {
    for (auto &p : tau.parts) parts.emplace(p.first, GPART(p.first, __nbatch, __gdims, p.second, fcode, _dev));
  }
  // transport
  SO3vec(const SO3vec &x, const int _dev) : _nbatch(x._nbatch), _gdims(x._gdims), dev(_dev) {
    for (auto &p : x.parts) parts.emplace(p.first, GPART(p.second, _dev));
  }

  int getb() const { return _nbatch; }
  Gdims get_gdims() const { return _gdims; }
  int get_dev() const { return dev; }
  int dominant_batch(const SO3vec &y) const { return std::max(_nbatch, y._nbatch); }
  Gdims dominant_gdims(const SO3vec &y) const { return _gdims.size() ? _gdims : y._gdims; }
  bool has_part(const int l) const { return parts.find(l) != parts.end(); }
  GPART &part(const int l) const { return parts.at(l); }
  GPART &operator[](const int l) const { return parts.at(l); }
  SO3type get_tau() const {
    SO3type R;
    for (auto &p : parts) R[p.first] = p.second.getn();
    return R;
  }

  // value-returning products (core/Gvec.hpp:296-301, 351-356); `limit` keeps only l <= limit
  SO3vec CGproduct(const SO3vec &y, const int limit = -1) const {
    SO3vec R(dominant_batch(y), dominant_gdims(y), get_tau().CGproduct(y.get_tau(), limit), 0, dev);
    R.add_CGproduct(*this, y);
    return R;
  }
  SO3vec DiagCGproduct(const SO3vec &y, const int limit = -1) const {
    SO3vec R(dominant_batch(y), dominant_gdims(y), get_tau().DiagCGproduct(y.get_tau(), limit), 0, dev);
    R.add_DiagCGproduct(*this, y);
    return R;
  }

  // One fused launch per call instead of the reference's launch per (l1,l2,l) triple (core/Gvec.hpp:311-389);
  // block layout and offsets are the reference's.
  void add_CGproduct(const SO3vec &x, const SO3vec &y) { fwd(false, x, y); }
  void add_CGproduct_back0(const SO3vec &g, const SO3vec &y) { bwd(false, this, nullptr, g, *this, y); }
  void add_CGproduct_back1(const SO3vec &g, const SO3vec &x) { bwd(false, nullptr, this, g, x, *this); }
  void add_DiagCGproduct(const SO3vec &x, const SO3vec &y) { fwd(true, x, y); }
  void add_DiagCGproduct_back0(const SO3vec &g, const SO3vec &y) { bwd(true, this, nullptr, g, *this, y); }
  void add_DiagCGproduct_back1(const SO3vec &g, const SO3vec &x) { bwd(true, nullptr, this, g, x, *this); }
  // both gradients from one pass over g (no counterpart in the reference, which reads g twice)
  static void add_CGproduct_back(SO3vec &xg, SO3vec &yg, const SO3vec &g, const SO3vec &x, const SO3vec &y) {
    bwd(false, &xg, &yg, g, x, y);
  }
  static void add_DiagCGproduct_back(SO3vec &xg, SO3vec &yg, const SO3vec &g, const SO3vec &x, const SO3vec &y) {
    bwd(true, &xg, &yg, g, x, y);
  }

  std::string classname() const { return "GElib::SO3vec"; }
  std::string repr() const { return "<GElib::SO3vec of type " + get_tau().str() + " [b=" + std::to_string(_nbatch) + "]>"; }
  std::string str(const std::string indent = "") const { return indent + repr(); }

 private:
  static std::vector<gelib_part_desc> descs(const SO3vec &v) {
    std::vector<gelib_part_desc> d;
    for (auto &p : v.parts) d.push_back(p.second.descriptor());
    return d;
  }
  static void on_gpu(const SO3vec &v) {
    for (auto &p : v.parts)
      if (p.second.get_dev() != 1) GELIB_ERROR("SO3vec must be on GPU: products of host parts are not part of this build");
  }
  void fwd(const bool diag, const SO3vec &x, const SO3vec &y) {
    on_gpu(*this), on_gpu(x), on_gpu(y);
    auto R = descs(*this), X = descs(x), Y = descs(y);
    auto fn = diag ? gelib_hip_so3vec_diagcg_fwd : gelib_hip_so3vec_cg_fwd;
    detail::skip_on(fn((int)R.size(), R.data(), (int)X.size(), X.data(), (int)Y.size(), Y.data(), accumulate_mode(), gelib_stream()));
  }
  static void bwd(const bool diag, const SO3vec *xg, const SO3vec *yg, const SO3vec &g, const SO3vec &x, const SO3vec &y) {
    on_gpu(g), on_gpu(x), on_gpu(y);
    std::vector<gelib_part_desc> XG, YG;
    if (xg) XG = descs(*xg);
    if (yg) YG = descs(*yg);
    auto G = descs(g), X = descs(x), Y = descs(y);
    auto fn = diag ? gelib_hip_so3vec_diagcg_bwd : gelib_hip_so3vec_cg_bwd;
    detail::skip_on(fn(xg ? XG.data() : nullptr, yg ? YG.data() : nullptr, (int)G.size(), G.data(), (int)X.size(), X.data(),
                       (int)Y.size(), Y.data(), accumulate_mode(), gelib_stream()));
  }
};

template <typename GVEC, typename... Args>
typename std::enable_if<std::is_base_of<GvecBase, GVEC>::value, GVEC>::type CGproduct(const GVEC &x, const GVEC &y,
                                                                                      const Args &...args) {
  return x.CGproduct(y, args...);
}
template <typename GVEC, typename... Args>
typename std::enable_if<std::is_base_of<GvecBase, GVEC>::value, GVEC>::type DiagCGproduct(const GVEC &x, const GVEC &y,
                                                                                          const Args &...args) {
  return x.DiagCGproduct(y, args...);
}

}  // namespace GElib
