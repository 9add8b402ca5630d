// PyTorch extension module `gelib_base`: the pybind11 surface of the reference's extension for the
// Clebsch-Gordan product path (python/bindings/GElib_py.cpp:46-74, SO3part_py.cpp:15-58, SO3vec_py.cpp:15-60,
// SO3type_py.cpp:16-44), rebuilt against PyTorch-ROCm over the C++ mirror in include/gelib/GElib.hpp.
// Tensors are aliased, never copied (python/bindings/SO3part_py.cpp:18-19); every product is queued on torch's
// current HIP stream.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include <pybind11/complex.h>
#include <pybind11/stl.h>

#include "gelib/GElib.hpp"

namespace py = pybind11;
using namespace GElib;

typedef cnine::TensorView<std::complex<float>> tensorc;

// zero-copy view of a complex64 tensor; dev 0 = host, 1 = GPU
static tensorc view_of(const at::Tensor &x) {
  TORCH_CHECK(x.scalar_type() == at::kComplexFloat, "GElib: SO3parts are complex64 tensors");
  cnine::Gdims dims;
  std::vector<size_t> strides;
  for (int i = 0; i < x.dim(); i++) {
    dims.push_back((int)x.size(i));
    TORCH_CHECK(x.stride(i) >= 0, "GElib: negative strides are not supported");
    strides.push_back((size_t)x.stride(i));
  }
  return tensorc(reinterpret_cast<std::complex<float> *>(x.data_ptr()), dims, cnine::GstridesB(strides), x.is_cuda() ? 1 : 0);
}

struct StreamGuard {  // products go to torch's current stream of the tensor's device
  explicit StreamGuard(int accumulate = 1) {
    try {
      gelib_stream() = (void *)c10::hip::getCurrentHIPStream().stream();
    } catch (const c10::Error &) {
      gelib_stream() = nullptr;  // no GPU: the dispatcher below reports "must be on GPU" for host tensors
    }
    accumulate_mode() = accumulate;
  }
  ~StreamGuard() {
    gelib_stream() = nullptr;
    accumulate_mode() = 1;
  }
};

static SO3vec<float> vec_of(const std::vector<at::Tensor> &parts) {
  SO3vec<float> R;
  for (auto &p : parts) {
    auto P = view_of(p);
    R.parts.emplace((P.dim(-2) - 1) / 2, SO3part<float>(P));
  }
  if (R.parts.size() > 0) {
    auto &P = R.parts.begin()->second;
    R._nbatch = P.getb();
    R._gdims = P.get_gdims();
    R.dev = P.dev;
  }
  return R;
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("version", []() { return std::string(_GELIB_VERSION); });

  py::class_<SO3type>(m, "SO3type", "Class to store the type of an SO3-vector")
      .def(py::init<>())
      .def(py::init<std::vector<int>>())
      .def(py::init<std::map<int, int>>())
      .def("__len__", &SO3type::size)
      .def("maxl", &SO3type::highest)
      .def("__getitem__", &SO3type::operator())
      .def("__setitem__", &SO3type::set)
      .def("get_parts", [](const SO3type &x) { return x.parts; })
      .def("CGproduct", [](const SO3type &x, const SO3type &y) { return x.CGproduct(y, -1); })
      .def("CGproduct", [](const SO3type &x, const SO3type &y, int maxl) { return x.CGproduct(y, maxl); })
      .def("DiagCGproduct", [](const SO3type &x, const SO3type &y) { return x.DiagCGproduct(y, -1); })
      .def("DiagCGproduct", [](const SO3type &x, const SO3type &y, int maxl) { return x.DiagCGproduct(y, maxl); })
      .def("str", &SO3type::str, py::arg("indent") = "")
      .def("__str__", &SO3type::str, py::arg("indent") = "")
      .def("__repr__", &SO3type::repr);
  m.def("CGproduct", [](const SO3type &x, const SO3type &y) { return x.CGproduct(y, -1); });
  m.def("CGproduct", [](const SO3type &x, const SO3type &y, const int maxl) { return x.CGproduct(y, maxl); });

  // python/bindings/gather_map_py.cpp:15-29
  py::class_<cnine::GatherMapB>(m, "gather_map", "A list of (source, target) pairs for sums of slices")
      .def_static("sources_targets",
                  [](const std::vector<int> sources, const std::vector<int> targets, int n_in, int n_out) {
                    return cnine::GatherMapB(sources, targets, n_in, n_out);
                  },
                  py::arg("sources"), py::arg("targets"), py::arg("n_in") = -1, py::arg("n_out") = -1)
      .def_static("from_matrix",
                  [](const at::Tensor &M, const int nin, const int nout) {
                    TORCH_CHECK(M.scalar_type() == at::kInt && M.dim() == 2 && !M.is_cuda(),
                                "GElib: a gather map is built from a k x 2 int32 host tensor of (source, target) rows");
                    cnine::Gdims dims;
                    std::vector<size_t> strides;
                    for (int i = 0; i < 2; i++) dims.push_back((int)M.size(i)), strides.push_back((size_t)M.stride(i));
                    return cnine::GatherMapB(cnine::TensorView<int>(M.data_ptr<int>(), dims, cnine::GstridesB(strides), 0), nin, nout);
                  })
      .def_static("random", [](const int n, const int m, const float p, unsigned seed) { return cnine::GatherMapB::random(n, m, p, seed); },
                  py::arg("n"), py::arg("m"), py::arg("p") = 0.5, py::arg("seed") = 0)
      .def("inv", &cnine::GatherMapB::inv)
      .def("d_in", &cnine::GatherMapB::d_in)
      .def("d_out", &cnine::GatherMapB::d_out)
      .def("pairs", [](const cnine::GatherMapB &g) { return g.inverted ? std::make_pair(g.targets, g.sources) : std::make_pair(g.sources, g.targets); })
      .def("str", &cnine::GatherMapB::str, py::arg("indent") = "")
      .def("__str__", &cnine::GatherMapB::str, py::arg("indent") = "")
      .def("__repr__", &cnine::GatherMapB::repr);

  py::class_<SO3part<float>>(m, "SO3part",
                             "n vectors transforming according to one irreducible representation of SO(3)")
      .def_static("view", [](at::Tensor &x) { return SO3part<float>(view_of(x)); })
      .def("add_CGproduct",
           [](SO3part<float> &r, const SO3part<float> &x, const SO3part<float> &y, const int offs) {
             StreamGuard g;
             Gpart_add_CGproduct(r, x, y, offs);
           },
           py::arg("x"), py::arg("y"), py::arg("offs") = 0)
      .def("add_CGproduct_back0",
           [](SO3part<float> &r, SO3part<float> &g, const SO3part<float> &y, const int offs) {
             StreamGuard sg;
             Gpart_add_CGproduct_back0(r, g, y, offs);
           },
           py::arg("g"), py::arg("y"), py::arg("offs") = 0)
      .def("add_CGproduct_back1",
           [](SO3part<float> &r, SO3part<float> &g, const SO3part<float> &x, const int offs) {
             StreamGuard sg;
             Gpart_add_CGproduct_back1(r, g, x, offs);
           },
           py::arg("g"), py::arg("x"), py::arg("offs") = 0)
      .def("add_DiagCGproduct",
           [](SO3part<float> &r, const SO3part<float> &x, const SO3part<float> &y, const int offs) {
             StreamGuard g;
             Gpart_add_DiagCGproduct(r, x, y, offs);
           },
           py::arg("x"), py::arg("y"), py::arg("offs") = 0)
      .def("add_DiagCGproduct_back0",
           [](SO3part<float> &r, SO3part<float> &g, const SO3part<float> &y, const int offs) {
             StreamGuard sg;
             Gpart_add_DiagCGproduct_back0(r, g, y, offs);
           },
           py::arg("g"), py::arg("y"), py::arg("offs") = 0)
      .def("add_DiagCGproduct_back1",
           [](SO3part<float> &r, SO3part<float> &g, const SO3part<float> &x, const int offs) {
             StreamGuard sg;
             Gpart_add_DiagCGproduct_back1(r, g, x, offs);
           },
           py::arg("g"), py::arg("x"), py::arg("offs") = 0)
      .def("add_spharm",
           [](SO3part<float> &r, at::Tensor &X) {
             TORCH_CHECK(X.scalar_type() == at::kFloat, "GElib: add_spharm takes a float32 tensor of (x, y, z) vectors");
             cnine::Gdims dims;
             std::vector<size_t> strides;
             for (int i = 0; i < X.dim(); i++) {
               dims.push_back((int)X.size(i));
               TORCH_CHECK(X.stride(i) >= 0, "GElib: negative strides are not supported");
               strides.push_back((size_t)X.stride(i));
             }
             StreamGuard sg;
             r.add_spharm(cnine::TensorView<float>(X.data_ptr<float>(), dims, cnine::GstridesB(strides), X.is_cuda() ? 1 : 0));
           },
           py::arg("X"))
      .def("add_gather",
           [](SO3part<float> &r, at::Tensor &x, const cnine::GatherMapB &gmap, int d) {
             StreamGuard sg;
             r.add_gather(SO3part<float>(view_of(x)), gmap, d);
           },
           py::arg("x"), py::arg("gmap"), py::arg("d") = 0)
      .def("add_gather_back",
           [](SO3part<float> &xg, at::Tensor &rg, const cnine::GatherMapB &gmap, int d) {
             StreamGuard sg;
             xg.add_gather_back(SO3part<float>(view_of(rg)), gmap, d);
           },
           py::arg("rg"), py::arg("gmap"), py::arg("d") = 0)
      .def("getl", &SO3part<float>::getl)
      .def("getn", &SO3part<float>::getn)
      .def("str", &SO3part<float>::str, py::arg("indent") = "")
      .def("__str__", &SO3part<float>::str, py::arg("indent") = "")
      .def("__repr__", &SO3part<float>::repr);

  // value-returning product of two parts; the result is a fresh torch tensor
  m.def("CGproduct", [](at::Tensor &x, at::Tensor &y, const int l) {
    SO3part<float> X(view_of(x)), Y(view_of(y));
    GELIB_ASSRT(SO3group::CGmultiplicity(X.getl(), Y.getl(), l) > 0);
    std::vector<int64_t> shape(x.sizes().begin(), x.sizes().end());
    if (y.dim() > x.dim()) shape.assign(y.sizes().begin(), y.sizes().end());
    shape[0] = std::max(x.size(0), y.size(0));
    shape[shape.size() - 2] = 2 * l + 1;
    shape[shape.size() - 1] = x.size(-1) * y.size(-1);
    at::Tensor r = at::zeros(shape, x.options());
    StreamGuard g;
    Gpart_add_CGproduct(SO3part<float>(view_of(r)), X, Y, 0);
    return r;
  });

  py::class_<SO3vec<float>>(m, "SO3vec", "Class to store an SO(3)-covariant vector")
      .def_static("view",
                  [](std::map<int, at::Tensor> &parts) {
                    std::vector<at::Tensor> v;
                    for (auto &p : parts) v.push_back(p.second);
                    return vec_of(v);
                  })
      .def_static("view", [](std::vector<at::Tensor> &parts) { return vec_of(parts); })
      .def("get_tau", &SO3vec<float>::get_tau)
      .def("addCGproduct",
           [](SO3vec<float> &r, const SO3vec<float> &x, const SO3vec<float> &y) {
             StreamGuard g;
             r.add_CGproduct(x, y);
           },
           py::arg("x"), py::arg("y"))
      .def("addCGproduct_back0",
           [](SO3vec<float> &r, const SO3vec<float> &g, const SO3vec<float> &y) {
             StreamGuard sg;
             r.add_CGproduct_back0(g, y);
           },
           py::arg("g"), py::arg("y"))
      .def("addCGproduct_back1",
           [](SO3vec<float> &r, const SO3vec<float> &g, const SO3vec<float> &x) {
             StreamGuard sg;
             r.add_CGproduct_back1(g, x);
           },
           py::arg("g"), py::arg("x"))
      .def("addDiagCGproduct",
           [](SO3vec<float> &r, const SO3vec<float> &x, const SO3vec<float> &y) {
             StreamGuard g;
             r.add_DiagCGproduct(x, y);
           },
           py::arg("x"), py::arg("y"))
      .def("addDiagCGproduct_back0",
           [](SO3vec<float> &r, const SO3vec<float> &g, const SO3vec<float> &y) {
             StreamGuard sg;
             r.add_DiagCGproduct_back0(g, y);
           },
           py::arg("g"), py::arg("y"))
      .def("addDiagCGproduct_back1",
           [](SO3vec<float> &r, const SO3vec<float> &g, const SO3vec<float> &x) {
             StreamGuard sg;
             r.add_DiagCGproduct_back1(g, x);
           },
           py::arg("g"), py::arg("x"))
      // One-pass variants without a counterpart in the reference: the product written into uninitialised parts
      // (no zero-fill, no read of r), and both gradients from a single pass over g.
      .def("setCGproduct",
           [](SO3vec<float> &r, const SO3vec<float> &x, const SO3vec<float> &y) {
             StreamGuard g(0);
             r.add_CGproduct(x, y);
           },
           py::arg("x"), py::arg("y"))
      .def("setDiagCGproduct",
           [](SO3vec<float> &r, const SO3vec<float> &x, const SO3vec<float> &y) {
             StreamGuard g(0);
             r.add_DiagCGproduct(x, y);
           },
           py::arg("x"), py::arg("y"))
      .def_static("setCGproduct_back",
                  [](SO3vec<float> &xg, SO3vec<float> &yg, const SO3vec<float> &g, const SO3vec<float> &x,
                     const SO3vec<float> &y) {
                    StreamGuard sg(0);
                    SO3vec<float>::add_CGproduct_back(xg, yg, g, x, y);
                  })
      .def_static("setDiagCGproduct_back",
                  [](SO3vec<float> &xg, SO3vec<float> &yg, const SO3vec<float> &g, const SO3vec<float> &x,
                     const SO3vec<float> &y) {
                    StreamGuard sg(0);
                    SO3vec<float>::add_DiagCGproduct_back(xg, yg, g, x, y);
                  })
      .def("str", &SO3vec<float>::str, py::arg("indent") = "")
      .def("__str__", &SO3vec<float>::str, py::arg("indent") = "")
      .def("__repr__", &SO3vec<float>::repr);
}
