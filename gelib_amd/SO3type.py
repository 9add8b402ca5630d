"""SO3type: {l: multiplicity}, a dict (python/src/gelib/SO3type.py:12-18), with the product rules of
core/Gtype.hpp:115-138 so that output types can be computed without touching a tensor."""
from gelib_amd.gelib_common import backend


class SO3type(dict):

    def CGproduct(self, y, maxl=-1):
        t = backend().SO3type(dict(self)).CGproduct(backend().SO3type(dict(y)), maxl)
        return SO3type(t.get_parts())

    def DiagCGproduct(self, y, maxl=-1):
        t = backend().SO3type(dict(self)).DiagCGproduct(backend().SO3type(dict(y)), maxl)
        return SO3type(t.get_parts())
