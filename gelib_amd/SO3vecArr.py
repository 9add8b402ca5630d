"""SO3vecArr: an array of SO(3)-covariant vectors, a dict {l: (b, a_1..a_k, 2l+1, n_l) complex64 tensor} -- the class
and autograd functions of python/src/gelib/SO3vecArr.py:23-401 for the CG product path.  The products are the same
fused launches as for SO3vec; the grid dimensions ride in the part descriptors."""
import torch

from gelib_amd.SO3weights import mix_channels
from gelib_amd.gelib_common import backend
from gelib_amd.SO3partArr import SO3partArr
from gelib_amd.SO3vec import _product_fn


class SO3vecArr:

    def __init__(self, *args):
        self.parts = {}
        if len(args) == 1 and not isinstance(args[0], torch.Tensor) and hasattr(args[0], '__iter__'):
            args = list(args[0])
        for x in args:
            assert isinstance(x, torch.Tensor)
            p = SO3partArr(x)
            self.parts[p.getl()] = x

    @classmethod
    def _filled(cls, maker, b, adims, tau, device):
        adims = [] if adims is None else list(adims)
        R = SO3vecArr()
        items = tau.items() if isinstance(tau, dict) else enumerate(tau)
        for l, n in items:
            R.parts[l] = maker(b, adims, l, n, device=device)
        return R

    @classmethod
    def zeros(cls, b, adims, tau, device='cpu'):
        return cls._filled(SO3partArr.zeros, b, adims, tau, device)

    @classmethod
    def ones(cls, b, adims, tau, device='cpu'):
        return cls._filled(SO3partArr.ones, b, adims, tau, device)

    @classmethod
    def randn(cls, b, adims, tau, device='cpu'):
        return cls._filled(SO3partArr.randn, b, adims, tau, device)

    @classmethod
    def zeros_like(cls, x):
        R = SO3vecArr()
        for l, p in x.parts.items():
            R.parts[l] = SO3partArr(torch.zeros_like(p))
        return R

    @classmethod
    def randn_like(cls, x):
        R = SO3vecArr()
        for l, p in x.parts.items():
            R.parts[l] = SO3partArr.randn_like(p)
        return R

    def backend(self):
        return backend().SO3vec.view(self.parts)

    def getb(self):
        if not self.parts:
            return 0
        return next(iter(self.parts.values())).size(0)

    def get_adims(self):
        if not self.parts:
            return []
        p = self.parts[min(self.parts)]
        return list(p.size()[1:p.dim() - 2])

    def tau(self):
        return {l: p.size(-1) for l, p in self.parts.items()}

    get_type = tau

    def l_max(self):
        return max(self.parts.keys()) if self.parts else 0

    def requires_grad_(self):
        for p in self.parts.values():
            p.requires_grad_()

    def get_grad(self):
        return SO3vecArr(*[p.grad for p in self.parts.values()])

    def apply(self, R):
        r = SO3vecArr()
        for l, p in self.parts.items():
            r.parts[l] = SO3partArr(p).apply(R)
        return r

    def gather(self, gmap, dim=0):
        """Part by part (python/src/gelib/SO3vecArr.py:230-234)."""
        return SO3vecArr(*[SO3partArr(p).gather(gmap, dim) for p in self.parts.values()])

    def odot(self, y):
        assert list(self.parts.keys()) == list(y.parts.keys())
        return sum(SO3partArr(self.parts[l]).odot(y.parts[l]) for l in self.parts.keys())

    def __add__(self, y):
        assert list(self.parts.keys()) == list(y.parts.keys())
        return SO3vecArr(*[self.parts[l] + y.parts[l] for l in self.parts.keys()])

    def to(self, device, non_blocking=False, copy=False, memory_format=torch.preserve_format):
        r = SO3vecArr()
        for l, p in self.parts.items():
            r.parts[l] = p.to(device, non_blocking=non_blocking, copy=copy, memory_format=memory_format)
        return r

    @property
    def device(self):
        if not self.parts:
            return torch.device("cpu")
        return next(iter(self.parts.values())).device

    @property
    def dtype(self):
        return self.parts[min(self.parts)].dtype if self.parts else torch.cfloat

    def __mul__(self, y):
        """Multiply every part by the matching weight matrix of an SO3weights (python/src/gelib/SO3vec.py:174-177)."""
        return SO3vecArr(*[mix_channels(p, w) for p, w in zip(self.parts.values(), y.parts)])

    def CGproduct(self, y, maxl=-1):
        assert isinstance(y, SO3vecArr)
        maxl = -1 if maxl is None else maxl
        xparts = list(self.parts.values())
        yparts = list(y.parts.values())
        return SO3vecArr(*SO3vecArr_CGproductFn.apply(len(xparts), len(yparts), maxl, *(xparts + yparts)))

    def DiagCGproduct(self, y, maxl=-1):
        assert isinstance(y, SO3vecArr)
        maxl = -1 if maxl is None else maxl
        xparts = list(self.parts.values())
        yparts = list(y.parts.values())
        return SO3vecArr(*SO3vecArr_DiagCGproductFn.apply(len(xparts), len(yparts), maxl, *(xparts + yparts)))

    def __repr__(self):
        return "<SO3vecArr of type %s [b=%d, adims=%s]>" % (self.tau(), self.getb(), self.get_adims())


SO3vecArr_CGproductFn = _product_fn(False, SO3partArr, "SO3vecArr")
SO3vecArr_DiagCGproductFn = _product_fn(True, SO3partArr, "SO3vecArr")
