// Minimal stand-in for the parts of the cnine tensor library that GElib's Clebsch-Gordan product path touches.
//
// GElib's headers build on cnine (include/GElib_base.hpp:17-19, core/Gpart.hpp:19-24); the members listed here are
// the ones that path uses: TensorView with public arr / dims / strides / dev, value copies that alias the same
// memory (core/CGproduct.hpp:45 passes parts by value and the caller sees the result), the fill codes 0 (zero)
// and 4 (gaussian) of SO3/tests/testSO3part.cpp:20,31, transport between host (dev 0) and GPU0 (dev 1) as in
// SO3/SO3part.hpp:182-183, slice / fuse helpers of core/Gpart.hpp, and BatchedTensor::getb.
// Device memory goes through the C ABI of libgelib_hip.so, so this header needs no HIP headers.
#pragma once

#include <cassert>
#include <complex>
#include <cstdint>
#include <cstring>
#include <initializer_list>
#include <memory>
#include <random>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "gelib_hip.h"

namespace cnine {

inline int roundup(const int x, const int s) { return ((x - 1) / s + 1) * s; }

template <typename T>
inline T ifthen(const bool c, const T &a, const T &b) {
  return c ? a : b;
}

class Gdims : public std::vector<int> {
 public:
  Gdims() {}
  Gdims(const std::initializer_list<int> &l) : std::vector<int>(l) {}
  Gdims(const std::vector<int> &v) : std::vector<int>(v) {}
  explicit Gdims(const int k) : std::vector<int>(k, 0) {}
  // (b, grid..., tail...)
  Gdims(const int b, const Gdims &g, const std::initializer_list<int> &tail) {
    push_back(b);
    for (auto v : g) push_back(v);
    for (auto v : tail) push_back(v);
  }
  int operator()(const int i) const { return i < 0 ? (*this)[size() + i] : (*this)[i]; }
  int last() const { return back(); }
  Gdims chunk(const int beg, int n = -1) const {
    if (n < 0) n = (int)size() - beg;
    Gdims r;
    for (int i = 0; i < n; i++) r.push_back((*this)[beg + i]);
    return r;
  }
  Gdims copy() const { return *this; }
  Gdims &set_back(const int i, const int v) {  // i-th from the back
    (*this)[size() - 1 - i] = v;
    return *this;
  }
  size_t total() const {
    size_t t = 1;
    for (auto v : *this) t *= (size_t)v;
    return t;
  }
  std::string str() const {
    std::ostringstream oss;
    oss << "(";
    for (size_t i = 0; i < size(); i++) oss << (*this)[i] << (i + 1 < size() ? "," : "");
    oss << ")";
    return oss.str();
  }
};

inline Gdims dims(const int a, const int b) { return Gdims({a, b}); }

class GstridesB : public std::vector<size_t> {
 public:
  GstridesB() {}
  GstridesB(const std::initializer_list<size_t> &l) : std::vector<size_t>(l) {}
  GstridesB(const std::vector<size_t> &v) : std::vector<size_t>(v) {}
  // packed row-major strides of dims
  explicit GstridesB(const Gdims &d) : std::vector<size_t>(d.size()) {
    size_t s = 1;
    for (int i = (int)d.size() - 1; i >= 0; i--) {
      (*this)[i] = s;
      s *= (size_t)d[i];
    }
  }
  GstridesB chunk(const int beg, int n = -1) const {
    if (n < 0) n = (int)size() - beg;
    GstridesB r;
    for (int i = 0; i < n; i++) r.push_back((*this)[beg + i]);
    return r;
  }
};

// Owner of a host or device allocation; TensorViews share it.
class MemBlock {
 public:
  void *ptr = nullptr;
  int dev = 0;
  MemBlock(const size_t bytes, const int _dev) : dev(_dev) {
    if (dev == 0) {
      ptr = ::operator new(bytes ? bytes : 1);
    } else {
      int rc = gelib_hip_malloc(&ptr, bytes);
      if (rc) throw std::runtime_error(std::string("cnine: device allocation failed: ") + gelib_hip_strerror(rc));
    }
  }
  ~MemBlock() {
    if (dev == 0) ::operator delete(ptr);
    else (void)gelib_hip_free(ptr);
  }
  MemBlock(const MemBlock &) = delete;
  MemBlock &operator=(const MemBlock &) = delete;
};

template <typename TYPE>
class TensorView {
 public:
  TYPE *arr = nullptr;
  Gdims dims;
  GstridesB strides;
  int dev = 0;
  std::shared_ptr<MemBlock> owner;  // empty for views of memory owned elsewhere (e.g. a torch tensor)

  TensorView() {}

  // non-owning view
  TensorView(TYPE *_arr, const Gdims &_dims, const GstridesB &_strides, const int _dev = 0)
      : arr(_arr), dims(_dims), strides(_strides), dev(_dev) {}

  // fcode 0: zeros, 4: iid gaussian (real and imaginary parts N(0,1) for complex types)
  TensorView(const Gdims &_dims, const int fcode = 0, const int _dev = 0) : dims(_dims), strides(_dims), dev(_dev) {
    const size_t n = dims.total();
    owner = std::make_shared<MemBlock>(n * sizeof(TYPE), dev);
    arr = static_cast<TYPE *>(owner->ptr);
    if (fcode == 0) {
      if (dev == 0) std::memset((void *)arr, 0, n * sizeof(TYPE));
      else check(gelib_hip_memset(arr, 0, n * sizeof(TYPE)));
      return;
    }
    std::vector<TYPE> host(n);
    fill_gaussian(host);
    if (dev == 0) std::memcpy((void *)arr, host.data(), n * sizeof(TYPE));
    else check(gelib_hip_memcpy(arr, host.data(), n * sizeof(TYPE), 0));
  }

  // transport: a packed copy of x on device _dev
  TensorView(const TensorView &x, const int _dev) : dims(x.dims), strides(x.dims), dev(_dev) {
    const size_t n = dims.total();
    owner = std::make_shared<MemBlock>(n * sizeof(TYPE), dev);
    arr = static_cast<TYPE *>(owner->ptr);
    TensorView px = x.packed();
    const int kind = (px.dev == 0 && dev == 1) ? 0 : (px.dev == 1 && dev == 0) ? 1 : (px.dev == 1 ? 2 : -1);
    if (kind < 0) std::memcpy((void *)arr, px.arr, n * sizeof(TYPE));
    else check(gelib_hip_memcpy(arr, px.arr, n * sizeof(TYPE), kind));
  }

  static unsigned &seed() {
    static unsigned s = 1;
    return s;
  }

  int get_dev() const { return dev; }
  TYPE *get_arr() const { return arr; }
  int ndims() const { return (int)dims.size(); }
  int dim(const int i) const { return dims(i); }
  size_t asize() const { return dims.total(); }
  bool is_packed() const {
    GstridesB p(dims);
    for (size_t i = 0; i < dims.size(); i++)
      if (dims[i] > 1 && p[i] != strides[i]) return false;
    return true;
  }

  // host access
  TYPE operator()(const int i0, const int i1) const {
    assert(dev == 0);
    return arr[i0 * strides[0] + i1 * strides[1]];
  }
  TYPE operator()(const int i0, const int i1, const int i2) const {
    assert(dev == 0);
    return arr[i0 * strides[0] + i1 * strides[1] + i2 * strides[2]];
  }
  void set(const int i0, const int i1, const int i2, const TYPE v) const {
    assert(dev == 0);
    arr[i0 * strides[0] + i1 * strides[1] + i2 * strides[2]] = v;
  }
  void inc(const int i0, const int i1, const TYPE v) const {
    assert(dev == 0);
    arr[i0 * strides[0] + i1 * strides[1]] += v;
  }

  TensorView slice(const int d, const int i) const {
    TensorView r(*this);
    r.arr = arr + (size_t)i * strides[d];
    r.dims.erase(r.dims.begin() + d);
    r.strides.erase(r.strides.begin() + d);
    return r;
  }

  TensorView zeros_like() const { return TensorView(dims, 0, dev); }

  // packed host-or-device copy with the same dev (a view of itself if already packed)
  TensorView packed() const {
    if (is_packed()) return *this;
    if (dev != 0) throw std::runtime_error("cnine: packing a strided device view is not supported");
    TensorView r(dims, 0, 0);
    std::vector<int> ix(dims.size(), 0);
    const size_t n = dims.total();
    for (size_t t = 0; t < n; t++) {
      size_t src = 0;
      for (size_t k = 0; k < dims.size(); k++) src += (size_t)ix[k] * strides[k];
      r.arr[t] = arr[src];
      for (int k = (int)dims.size() - 1; k >= 0; k--) {
        if (++ix[k] < dims[k]) break;
        ix[k] = 0;
      }
    }
    return r;
  }

  std::string dtype_str() const { return sizeof(TYPE) == 8 ? "complex<float>" : "other"; }
  std::string str(const std::string indent = "") const {
    std::ostringstream oss;
    oss << indent << "TensorView" << dims.str() << " on dev " << dev;
    return oss.str();
  }

 private:
  static void check(const int rc) {
    if (rc) throw std::runtime_error(std::string("cnine: ") + gelib_hip_strerror(rc) + " " + gelib_hip_last_runtime_error());
  }
  static void fill_gaussian(std::vector<std::complex<float>> &h) {
    std::mt19937 gen(seed()++);
    std::normal_distribution<float> d(0.f, 1.f);
    for (auto &v : h) v = std::complex<float>(d(gen), d(gen));
  }
  static void fill_gaussian(std::vector<float> &h) {
    std::mt19937 gen(seed()++);
    std::normal_distribution<float> d(0.f, 1.f);
    for (auto &v : h) v = d(gen);
  }
};

template <typename TYPE>
class BatchedTensor : public TensorView<TYPE> {
 public:
  using TensorView<TYPE>::TensorView;
  using TensorView<TYPE>::dims;
  BatchedTensor() {}
  BatchedTensor(const TensorView<TYPE> &x) : TensorView<TYPE>(x) {}
  int getb() const { return dims[0]; }
};

}  // namespace cnine
