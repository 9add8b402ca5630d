"""SO3partArr: an array of SO3parts, shape (b, a_1, ..., a_k, 2l+1, n) complex64 -- the class and autograd functions
of python/src/gelib/SO3partArr.py:18-234 for the CG product path.  The grid dimensions a_1..a_k travel to the kernels
as the grid dimensions of the part descriptor (core/Gpart.hpp:416-432, 495-531); nothing is reshaped or copied."""
import torch

from gelib_amd.gelib_common import backend, common_batch
from gelib_amd.SO3element import SO3element, SO3irrep
from gelib_amd.SO3part import SO3part


class SO3partArr(torch.Tensor):

    @staticmethod
    def zeros(b, adims, l, n, device='cpu'):
        return SO3partArr(torch.zeros([b] + list(adims) + [2 * l + 1, n], dtype=torch.complex64, device=device))

    @staticmethod
    def ones(b, adims, l, n, device='cpu'):
        return SO3partArr(torch.ones([b] + list(adims) + [2 * l + 1, n], dtype=torch.complex64, device=device))

    @staticmethod
    def randn(b, adims, l, n, device='cpu'):
        return SO3partArr(torch.randn([b] + list(adims) + [2 * l + 1, n], dtype=torch.complex64, device=device))

    @classmethod
    def spharm(cls, l, X):
        """Spherical harmonics of the vectors (x, y, z) in X, shaped (b, a_1..a_k, 3, n) float32
        (python/src/gelib/SO3partArr.py:59-67)."""
        assert X.size(-2) == 3
        R = SO3partArr.zeros(X.size(0), list(X.size())[1:X.dim() - 2], l, X.size(-1), device=X.device)
        R.backend().add_spharm(X)
        return R

    def zeros_like(self, *args):
        if not args:
            return SO3partArr(torch.zeros_like(self))
        assert len(args) == 2 and isinstance(args[0], int) and isinstance(args[1], int)
        dims = list(self.size())
        dims[-2], dims[-1] = 2 * args[0] + 1, args[1]
        return SO3partArr(torch.zeros(dims, dtype=torch.complex64, device=self.device))

    @classmethod
    def randn_like(cls, x):
        return SO3partArr(torch.randn_like(x))

    def backend(self):
        return backend().SO3part.view(self)

    def collapse(self):
        return SO3part(self.reshape(self.size(0), -1, self.size(-2), self.size(-1)))

    def getb(self):
        return self.size(0)

    def get_adims(self):
        return list(self.size()[1:self.dim() - 2])

    def get_nadims(self):
        return self.dim() - 3

    def getl(self):
        return int((self.size(-2) - 1) / 2)

    def getn(self):
        return self.size(-1)

    def odot(self, y):
        return torch.Tensor(torch.sum(torch.mul(torch.view_as_real(self), torch.view_as_real(y))))

    def apply(self, R):
        assert isinstance(R, SO3element)
        rho = SO3irrep(self.getl())
        return SO3partArr(torch.matmul(rho.matrix(R).to(self.device), self))

    def gather(self, gmap, dim=0):
        """Sums of cells along grid dimension dim: cell t of the result = sum of the cells s of self over the pairs
        (s, t) of gmap (python/src/gelib/SO3partArr.py:142-146)."""
        return SO3partArr_GatherFn.apply(self, gmap, dim)

    def CGproduct(self, y, l):
        return SO3partArr_CGproductFn.apply(self, y, l)

    def DiagCGproduct(self, y, l):
        return SO3partArr_DiagCGproductFn.apply(self, y, l)


def _view(t):
    return backend().SO3part.view(t)


def _part_fn(diag):
    name = "DiagCGproduct" if diag else "CGproduct"

    class Fn(torch.autograd.Function):

        @staticmethod
        def forward(ctx, x, y, l):
            ctx.l = l
            ctx.save_for_backward(x, y)
            b = common_batch(x, y)
            a = x.get_adims() if isinstance(x, SO3partArr) else list(x.size()[1:x.dim() - 2])
            if diag:
                assert x.size(-1) == y.size(-1)
            r = SO3partArr.zeros(b, a, l, x.size(-1) if diag else x.size(-1) * y.size(-1), device=x.device)
            getattr(_view(r), "add_" + name)(_view(x), _view(y))
            return r

        @staticmethod
        def backward(ctx, g):
            x, y = ctx.saved_tensors
            g = g.contiguous()
            xg = torch.zeros_like(x)
            yg = torch.zeros_like(y)
            getattr(_view(xg), "add_%s_back0" % name)(_view(g), _view(y))
            getattr(_view(yg), "add_%s_back1" % name)(_view(g), _view(x))
            return xg, yg, None

    Fn.__name__ = "SO3partArr_%sFn" % name
    return Fn


SO3partArr_CGproductFn = _part_fn(False)
SO3partArr_DiagCGproductFn = _part_fn(True)


class SO3partArr_GatherFn(torch.autograd.Function):
    """python/src/gelib/SO3partArr.py:236-254: forward add_gather, backward add_gather_back with the same map."""

    @staticmethod
    def forward(ctx, x, gmap, d):
        from gelib_amd.gather_map import gather_map
        assert isinstance(gmap, gather_map)
        adims = list(x.size()[1:x.dim() - 2])
        assert 0 <= d < len(adims) and len(adims) <= 2, "gather runs along one of at most two grid dimensions"
        assert adims[d] == gmap.d_in()
        ctx.gmap, ctx.d, ctx.adims = gmap, d, list(adims)
        adims[d] = gmap.d_out()
        r = SO3partArr.zeros(x.size(0), adims, (x.size(-2) - 1) // 2, x.size(-1), device=x.device)
        _view(r).add_gather(x, gmap.obj, d)
        return r

    @staticmethod
    def backward(ctx, rg):
        xg = SO3partArr.zeros(rg.size(0), ctx.adims, (rg.size(-2) - 1) // 2, rg.size(-1), device=rg.device)
        _view(xg).add_gather_back(rg.contiguous(), ctx.gmap.obj, ctx.d)
        return xg, None, None
