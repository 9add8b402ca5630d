"""SO3part: a torch.Tensor subclass holding n vectors that transform by one irrep of SO(3), shape (b, 2l+1, n),
complex64 -- the class and autograd functions of python/src/gelib/SO3part.py:22-220 for the CG product path."""
import torch

from gelib_amd.gelib_common import backend, common_batch
from gelib_amd.SO3element import SO3element, SO3irrep


class SO3part(torch.Tensor):

    @classmethod
    def zeros(cls, b, l, n, device='cpu'):
        return SO3part(torch.zeros([b, 2 * l + 1, n], dtype=torch.complex64, device=device))

    @classmethod
    def randn(cls, b, l, n, device='cpu'):
        return SO3part(torch.randn([b, 2 * l + 1, n], dtype=torch.complex64, device=device))

    @classmethod
    def spharm(cls, l, X):
        """Spherical harmonics of the vectors (x, y, z) in X, shaped (b, 3, n) float32
        (python/src/gelib/SO3part.py:55-62)."""
        assert X.dim() == 3
        R = SO3part.zeros(X.size(0), l, X.size(2), device=X.device)
        R.backend().add_spharm(X)
        return R

    def zeros_like(self, *args):
        if not args:
            return SO3part(torch.zeros_like(self))
        dims = list(self.size())
        if len(args) == 2:
            dims[-2], dims[-1] = 2 * args[0] + 1, args[1]
        elif len(args) == 3:
            dims[0], dims[-2], dims[-1] = args[0], 2 * args[1] + 1, args[2]
        return SO3part(torch.zeros(dims, dtype=torch.complex64, device=self.device))

    @classmethod
    def randn_like(cls, x):
        return SO3part(torch.randn_like(x))

    def backend(self):
        return backend().SO3part.view(self)

    def getb(self):
        return self.size(0)

    def getl(self):
        return int((self.size(-2) - 1) / 2)

    def getn(self):
        return self.size(-1)

    def apply(self, R):
        assert isinstance(R, SO3element)
        rho = SO3irrep(self.getl())
        return SO3part(torch.matmul(rho.matrix(R).to(self.device), self))

    def odot(self, y):
        return torch.Tensor(torch.sum(torch.mul(torch.view_as_real(self), torch.view_as_real(y))))

    def CGproduct(self, y, l):
        assert isinstance(y, SO3part)
        assert isinstance(l, int)
        return SO3part_CGproductFn.apply(self, y, l)

    def DiagCGproduct(self, y, l):
        assert isinstance(y, SO3part)
        assert isinstance(l, int)
        return SO3part_DiagCGproductFn.apply(self, y, l)


def _view(t):
    return backend().SO3part.view(t)


class SO3part_CGproductFn(torch.autograd.Function):

    @staticmethod
    def forward(ctx, x, y, l):
        ctx.l = l
        ctx.save_for_backward(x, y)
        b = common_batch(x, y)
        r = SO3part.zeros(b, l, x.size(-1) * y.size(-1), device=x.device)
        _view(r).add_CGproduct(_view(x), _view(y))
        return r

    @staticmethod
    def backward(ctx, g):
        x, y = ctx.saved_tensors
        g = g.contiguous()
        # both gradients from ONE pass over g (the vector-level backward on one-part vectors); the reference makes two
        # calls, each of which reads g.  An operand shared by the batch (extent 1) gets the sum over the batch, formed
        # inside the library in a fixed order.
        gb = backend()
        xg = torch.empty_like(x, memory_format=torch.contiguous_format)
        yg = torch.empty_like(y, memory_format=torch.contiguous_format)
        vec = gb.SO3vec.view
        gb.SO3vec.setCGproduct_back(vec([xg]), vec([yg]), vec([g]), vec([x]), vec([y]))
        return xg, yg, None


class SO3part_DiagCGproductFn(torch.autograd.Function):

    @staticmethod
    def forward(ctx, x, y, l):
        ctx.l = l
        ctx.save_for_backward(x, y)
        b = common_batch(x, y)
        assert x.size(-1) == y.size(-1)
        r = SO3part.zeros(b, l, x.size(-1), device=x.device)
        _view(r).add_DiagCGproduct(_view(x), _view(y))
        return r

    @staticmethod
    def backward(ctx, g):
        x, y = ctx.saved_tensors
        g = g.contiguous()
        xg = torch.zeros_like(x)
        yg = torch.zeros_like(y)
        _view(xg).add_DiagCGproduct_back0(_view(g), _view(y))
        _view(yg).add_DiagCGproduct_back1(_view(g), _view(x))
        return xg, yg, None
