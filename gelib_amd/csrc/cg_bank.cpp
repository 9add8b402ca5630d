// Clebsch-Gordan coefficient bank: host evaluation and per-device cached uploads.
//
// Takes the place of GElib's process-global SO3_CGbank (SO3/SO3CGbank.hpp:26-95, include/GElib_base.cpp:20):
// same numbers (Racah's sum evaluated with lgamma in double, rounded to float on store, row-major
// (2l1+1) x (2l2+1)), but guarded by a mutex and keyed per device.
#include <cmath>
#include <cstring>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "cg_common.h"

namespace gelib_hip {

static inline double lfact(int n) { return std::lgamma((double)n + 1.0); }

double cg_coeff(int l1, int l2, int l, int m1, int m2) {
  const int m = m1 + m2;
  if (l < std::abs(l1 - l2) || l > l1 + l2 || std::abs(m1) > l1 || std::abs(m2) > l2 || std::abs(m) > l) return 0.0;
  // Racah: sqrt(2l+1) * Delta * sqrt(prod of (l_i +- m_i)!) * sum_t (-1)^t / (t! (t-t1)! (t-t2)! (t3-t)! (t4-t)! (t5-t)!)
  const int t1 = l2 - m1 - l, t2 = l1 + m2 - l, t3 = l1 + l2 - l, t4 = l1 - m1, t5 = l2 + m2;
  const int tmin = std::max(0, std::max(t1, t2));
  const int tmax = std::min(t3, std::min(t4, t5));
  // same association order as the reference so that the float-rounded tables are identical to its bank
  double log_a = (lfact(l1 + l2 - l) + lfact(l1 - l2 + l) + lfact(-l1 + l2 + l) - lfact(l1 + l2 + l + 1)) / 2;
  log_a += (lfact(l1 + m1) + lfact(l1 - m1) + lfact(l2 + m2) + lfact(l2 - m2) + lfact(l - m) + lfact(l + m)) / 2;
  double sum = 0.0;
  for (int t = tmin; t <= tmax; t++) {
    const double log_b = lfact(t) + lfact(t - t1) + lfact(t - t2) + lfact(t3 - t) + lfact(t4 - t) + lfact(t5 - t);
    const double term = std::exp(log_a - log_b);
    sum += (t & 1) ? -1.0 * term : term;
  }
  return std::sqrt((double)(2 * l + 1)) * sum;
}

void cg_matrix_host(int l1, int l2, int l, float *out) {
  const int L1 = 2 * l1 + 1, L2 = 2 * l2 + 1;
  std::memset(out, 0, sizeof(float) * (size_t)L1 * L2);
  for (int m1 = -l1; m1 <= l1; m1++)
    for (int m2 = std::max(-l2, -l - m1); m2 <= std::min(l2, l - m1); m2++)
      out[(m1 + l1) * L2 + (m2 + l2)] = (float)cg_coeff(l1, l2, l, m1, m2);
}

namespace {
std::mutex g_bank_mutex;
std::map<std::tuple<int, int, int, int>, float *> g_bank;  // (device, l1, l2, l) -> device table
}  // namespace

int cg_matrix_device(int l1, int l2, int l, const float **dptr) {
  int dev = 0;
  GELIB_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_bank_mutex);
  auto key = std::make_tuple(dev, l1, l2, l);
  auto it = g_bank.find(key);
  if (it != g_bank.end()) {
    *dptr = it->second;
    return GELIB_HIP_OK;
  }
  const size_t n = (size_t)(2 * l1 + 1) * (2 * l2 + 1);
  std::vector<float> host(n);
  cg_matrix_host(l1, l2, l, host.data());
  float *d = nullptr;
  GELIB_HIP_TRY(hipMalloc((void **)&d, n * sizeof(float)));
  // Synchronous copy: the table must be complete before any stream reads it.
  hipError_t e = hipMemcpy(d, host.data(), n * sizeof(float), hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    (void)hipFree(d);
    return record_hip_error(e, "hipMemcpy(cg table)");
  }
  g_bank.emplace(key, d);
  *dptr = d;
  return GELIB_HIP_OK;
}

}  // namespace gelib_hip
