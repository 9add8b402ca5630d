"""Builds the PyTorch extension module gelib_base in-tree (gelib_amd/gelib_base*.so).

    python gelib_amd/bindings/setup.py build_ext --inplace

Host-only C++ (the HIP kernels live in libgelib_hip.so, which this module links with an $ORIGIN rpath)."""
import os

from setuptools import setup
from torch.utils import cpp_extension as ce

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
PKG = os.path.join(ROOT, "gelib_amd")

ext = ce.CppExtension(
    name="gelib_amd.gelib_base",
    sources=[os.path.join(HERE, "gelib_base.cpp")],
    # the class mirror is header-only: the module must be rebuilt when any of these changes
    depends=[os.path.join(ROOT, "include", "gelib", "GElib.hpp"), os.path.join(ROOT, "include", "gelib", "cnine_min.hpp"),
             os.path.join(ROOT, "include", "gelib_hip.h")],
    include_dirs=[os.path.join(ROOT, "include"), "/opt/rocm/include"],
    define_macros=[("__HIP_PLATFORM_AMD__", "1"), ("USE_ROCM", "1")],
    extra_compile_args=["-O2", "-g0", "-std=c++17", "-Wno-unused-function"],
    library_dirs=[PKG, os.path.join(os.path.dirname(ce.__file__), "..", "lib")],
    libraries=["gelib_hip", "c10_hip", "torch_hip"],
    extra_link_args=["-Wl,-rpath,$ORIGIN", "-s"],
)

setup(name="gelib_amd_base", version="0.1", ext_modules=[ext], cmdclass={"build_ext": ce.BuildExtension.with_options(use_ninja=False)},
      script_args=["build_ext", "--inplace", "--force", "--build-temp", os.path.join(PKG, "csrc", "build", "pybind"),
                   "--build-lib", os.path.join(PKG, "csrc", "build", "pybind_lib")],
      packages=[])
