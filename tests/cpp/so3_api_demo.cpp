// Exercises the C++ mirror of GElib's interface (include/gelib/GElib.hpp) the way the reference's own smoke
// programs do (SO3/tests/testSO3part.cpp, test_SO3partG.cpp): gaussian parts, CGproduct on the GPU, results
// written to a file that the Python test compares with the CPU oracle.
//   usage: so3_api_demo <out.bin>
#include <cstdio>
#include <fstream>

#include "gelib/GElib.hpp"

using namespace cnine;
using namespace GElib;

static void dump(std::ofstream &f, const TensorView<std::complex<float>> &t) {
  TensorView<std::complex<float>> h(t, 0);
  int nd = h.ndims();
  f.write((const char *)&nd, sizeof(int));
  for (int i = 0; i < nd; i++) {
    int d = h.dims[i];
    f.write((const char *)&d, sizeof(int));
  }
  f.write((const char *)h.arr, h.asize() * sizeof(std::complex<float>));
}

int main(int argc, char **argv) {
  if (argc < 2) return 2;
  std::ofstream f(argv[1], std::ios::binary);
  const int b = 3;

  // part level: l1=2, l2=1 -> l=2, with the forward and both backward dispatchers
  SO3part<float> x(b, 2, 4, 4, 0), y(b, 1, 8, 4, 0);
  SO3part<float> xd(x, 1), yd(y, 1);
  SO3part<float> r = CGproduct(xd, yd, 2);
  SO3part<float> g(b, 2, 32, 4, 0);
  SO3part<float> gd(g, 1);
  SO3part<float> xg = xd.zeros_like(), yg = yd.zeros_like();
  Gpart_add_CGproduct_back0(xg, gd, yd);
  Gpart_add_CGproduct_back1(yg, gd, xd);
  SO3part<float> rdiag = DiagCGproduct(xd, SO3part<float>(SO3part<float>(b, 1, 4, 4, 0), 1), 3);
  dump(f, x), dump(f, y), dump(f, r), dump(f, g), dump(f, xg), dump(f, yg);

  // vec level: tau = (2,2,2) x (2,2,2), capped at l <= 2
  SO3type tau({{0, 2}, {1, 2}, {2, 2}});
  SO3vec<float> u(b, Gdims(), tau, 4, 0), v(b, Gdims(), tau, 4, 0);
  SO3vec<float> ud(u, 1), vd(v, 1);
  SO3vec<float> w = CGproduct(ud, vd, 2);
  for (auto &p : u.parts) dump(f, p.second);
  for (auto &p : v.parts) dump(f, p.second);
  for (auto &p : w.parts) dump(f, p.second);

  // type arithmetic known answers (python/docs/source/abandoned/SO3type.rst:28-41)
  SO3type t1({{0, 1}, {1, 1}, {2, 1}});
  if (!(CGproduct(t1, t1) == SO3type(std::vector<int>{3, 6, 6, 3, 1}))) return 3;
  if (!(CGproduct(t1, t1, 2) == SO3type(std::vector<int>{3, 6, 6}))) return 4;
  if (w.get_tau().str() != tau.CGproduct(tau, 2).str()) return 5;

  // error conventions: device mismatch and triangle violation throw
  int caught = 0;
  try {
    Gpart_add_CGproduct(r, x, yd);
  } catch (std::runtime_error &) { caught++; }
  try {
    CGproduct(xd, yd, 5);
  } catch (std::runtime_error &) { caught++; }
  try {
    SO3part<float> small(b, 2, 7, 0, 1);
    Gpart_add_CGproduct(small, xd, yd);
  } catch (std::runtime_error &) { caught++; }
  if (caught != 3) return 6;
  if (SO3_CGbank.get<float>(1, 2, 2).dims != Gdims({3, 5})) return 7;
  gelib_check(gelib_hip_synchronize());
  printf("so3_api_demo ok %s\n", r.repr().c_str());
  return 0;
}
