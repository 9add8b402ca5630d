"""MI355X-native Clebsch-Gordan product path with GElib's Python surface:

    import gelib_amd as gelib
    z = gelib.CGproduct(x, y, l)          # SO3parts
    w = gelib.CGproduct(u, v, maxl=4)     # SO3vecs (one fused HIP launch forward, one backward)

The arithmetic runs in hand-written HIP kernels (libgelib_hip.so) reached through the pybind11 module
gelib_amd.gelib_base; tensors must live on the GPU.  Nothing here falls back to another implementation.
"""
from gelib_amd.gelib_common import common_batch  # noqa: F401
from gelib_amd.SO3element import SO3element, SO3irrep  # noqa: F401
from gelib_amd.SO3type import SO3type  # noqa: F401
from gelib_amd.SO3part import SO3part, SO3part_CGproductFn, SO3part_DiagCGproductFn  # noqa: F401
from gelib_amd.SO3vec import SO3vec, SO3vec_CGproductFn, SO3vec_DiagCGproductFn  # noqa: F401
from gelib_amd.SO3partArr import SO3partArr, SO3partArr_CGproductFn, SO3partArr_DiagCGproductFn  # noqa: F401
from gelib_amd.SO3vecArr import SO3vecArr, SO3vecArr_CGproductFn, SO3vecArr_DiagCGproductFn  # noqa: F401
from gelib_amd.SO3weights import SO3weights, SO3linear, CGproduct_linear  # noqa: F401
from gelib_amd.gather_map import gather_map  # noqa: F401
from gelib_amd.O3 import O3element, O3irrep, O3type, O3part, O3vec, O3vec_CGproductFn, O3vec_DiagCGproductFn  # noqa: F401


def CGproduct(x, y, maxl=-1):
    return x.CGproduct(y, maxl)


def DiagCGproduct(x, y, maxl=-1):
    return x.DiagCGproduct(y, maxl)
