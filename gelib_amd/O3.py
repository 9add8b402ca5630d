"""O(3) wrappers: parts and vectors labelled by mu = (l, parity), the classes of python/src/gelib/O3part.py,
O3vec.py, O3type.py, O3element.py and O3irrep.py for the CG product path.

O(3) adds nothing to the arithmetic: a product of parts with parities p1, p2 is the SO(3) product, labelled p1*p2
(O3/O3group.hpp:38-53, O3/O3part.hpp:214-269 forward every kernel to SO3part).  So these classes only keep the labels,
check the parity rule and enumerate the (mu1, mu2, mu) triples of a vector product in the reference's order -- parts
sorted by the index 2l + (p == -1) (O3/O3index.hpp:28-31), then l ascending, each block at the running channel offset
of its output part (core/Gvec.hpp:311-321) -- and call the part-level HIP entry points with those offsets.  There is
one launch per triple, as in the reference; the fused single-launch kernels take one part per l and are not used here.
"""
import torch

from gelib_amd.gelib_common import backend, common_batch
from gelib_amd.SO3element import SO3element, SO3irrep


def _index(mu):
    return 2 * mu[0] + (mu[1] == -1)


def _check_mu(mu):
    assert isinstance(mu, tuple) and len(mu) == 2 and isinstance(mu[0], int) and mu[1] in (1, -1)


class O3element(torch.Tensor):
    """An orthogonal 3x3 matrix, determinant +1 or -1 (O3/O3element.hpp:45-58)."""

    @classmethod
    def identity(cls):
        return O3element(torch.eye(3))

    @classmethod
    def random(cls):
        q, r = torch.linalg.qr(torch.randn(3, 3, dtype=torch.float64))
        q = q * torch.sign(torch.diagonal(r))          # Haar on O(3): both determinants occur
        return O3element(q.to(torch.float32))

    def parity(self):
        return 1 if torch.det(torch.as_tensor(self, dtype=torch.float64)) >= 0 else -1

    def inv(self):
        return O3element(self.t())


class O3irrep:
    """D_(l,p)(R) = D_l(det(R) R) for p = +1, det(R) D_l(det(R) R) for p = -1 (O3/O3irrep.hpp:36-43)."""

    def __init__(self, l, p):
        _check_mu((l, p))
        self.l, self.p = l, p

    def matrix(self, R):
        det = O3element(torch.as_tensor(R)).parity()
        D = SO3irrep(self.l).matrix(SO3element(torch.as_tensor(R) * det))
        return D * det if self.p == -1 else D


class O3type(dict):
    """{(l, p): multiplicity}; product rules of core/Gtype.hpp:115-138 with O3group's components."""

    def _product(self, y, maxl, diag):
        out = {}
        for mu1 in sorted(self, key=_index):
            for mu2 in sorted(y, key=_index):
                if diag:
                    assert self[mu1] == y[mu2], "DiagCGproduct needs equal multiplicities"
                for l in range(abs(mu1[0] - mu2[0]), mu1[0] + mu2[0] + 1):
                    if maxl >= 0 and l > maxl:
                        continue
                    mu = (l, mu1[1] * mu2[1])
                    out[mu] = out.get(mu, 0) + (self[mu1] if diag else self[mu1] * y[mu2])
        return O3type({mu: out[mu] for mu in sorted(out, key=_index)})

    def CGproduct(self, y, maxl=-1):
        return self._product(y, maxl, False)

    def DiagCGproduct(self, y, maxl=-1):
        return self._product(y, maxl, True)


def _plain(t):
    return t.as_subclass(torch.Tensor) if isinstance(t, torch.Tensor) else t


class O3part(torch.Tensor):
    """(b, 2l+1, n) complex64 with the label mu = (l, p) (python/src/gelib/O3part.py:22-180).  Results of torch
    arithmetic on parts are parts without a label; the constructors and products of this module attach it."""

    def __new__(cls, T, mu):
        _check_mu(mu)
        assert T.size(-2) == 2 * mu[0] + 1
        R = T.as_subclass(cls)      # stays attached to the autograd graph
        R.mu = mu
        return R

    def __init__(self, T, mu):
        pass

    @classmethod
    def zeros(cls, b, mu, n, device='cpu'):
        return O3part(torch.zeros([b, 2 * mu[0] + 1, n], dtype=torch.complex64, device=device), mu)

    @classmethod
    def randn(cls, b, mu, n, device='cpu'):
        return O3part(torch.randn([b, 2 * mu[0] + 1, n], dtype=torch.complex64, device=device), mu)

    @classmethod
    def randn_like(cls, x):
        return O3part(torch.randn_like(_plain(x)), x.mu)

    def zeros_like(self):
        return O3part(torch.zeros_like(_plain(self)), self.mu)

    def backend(self):
        return backend().SO3part.view(_plain(self))

    def getb(self):
        return self.size(0)

    def get_mu(self):
        return self.mu

    def getp(self):
        return self.mu[1]

    def getl(self):
        return self.mu[0]

    def getn(self):
        return self.size(2)

    def apply(self, R):
        rho = O3irrep(self.getl(), self.getp())
        return O3part(torch.matmul(rho.matrix(R).to(self.device), _plain(self)), self.mu)

    def odot(self, y):
        return torch.sum(torch.mul(torch.view_as_real(_plain(self)), torch.view_as_real(_plain(y))))

    def CGproduct(self, y, mu):
        assert isinstance(y, O3part)
        return _part_product(self, y, mu, False)

    def DiagCGproduct(self, y, mu):
        assert isinstance(y, O3part)
        return _part_product(self, y, mu, True)


def _part_product(x, y, mu, diag):
    """python/src/gelib/O3part.py:189-236: the parity rule, then the SO(3) product of the same tensors."""
    from gelib_amd.SO3part import SO3part_CGproductFn, SO3part_DiagCGproductFn
    _check_mu(mu)
    assert x.getp() * y.getp() == mu[1], "the parity of a product is the product of the parities"
    fn = SO3part_DiagCGproductFn if diag else SO3part_CGproductFn
    return O3part(fn.apply(_plain(x), _plain(y), mu[0]), mu)


def _triples(xmus, ymus, rmus, ns_x, ns_y, diag):
    """(xi, yi, ri, offs) in the reference's order; offs = running channel offset inside output part ri."""
    offs = [0] * len(rmus)
    where = {mu: k for k, mu in enumerate(rmus)}
    out = []
    for xi, mu1 in enumerate(xmus):
        for yi, mu2 in enumerate(ymus):
            for l in range(abs(mu1[0] - mu2[0]), mu1[0] + mu2[0] + 1):
                mu = (l, mu1[1] * mu2[1])
                if mu not in where:
                    continue
                ri = where[mu]
                out.append((xi, yi, ri, offs[ri]))
                offs[ri] += ns_x[xi] if diag else ns_x[xi] * ns_y[yi]
    return out


def _vec_fn(diag):
    name = "DiagCGproduct" if diag else "CGproduct"

    class Fn(torch.autograd.Function):

        @staticmethod
        def forward(ctx, xmus, ymus, maxl, *args):
            gb = backend()
            k1 = len(xmus)
            xs, ys = args[:k1], args[k1:]
            tau = getattr(O3type({mu: t.size(-1) for mu, t in zip(xmus, xs)}), name)(
                O3type({mu: t.size(-1) for mu, t in zip(ymus, ys)}), maxl)
            b = common_batch(xs[0], ys[0])
            rmus = list(tau)
            rs = [torch.zeros([b, 2 * mu[0] + 1, n], dtype=torch.complex64, device=xs[0].device) for mu, n in tau.items()]
            ctx.triples = _triples(xmus, ymus, rmus, [t.size(-1) for t in xs], [t.size(-1) for t in ys], diag)
            ctx.k1, ctx.rmus = k1, rmus
            ctx.save_for_backward(*args)
            for xi, yi, ri, offs in ctx.triples:
                getattr(gb.SO3part.view(rs[ri]), "add_" + name)(gb.SO3part.view(xs[xi]), gb.SO3part.view(ys[yi]), offs)
            return tuple(rs)

        @staticmethod
        def backward(ctx, *gs):
            gb = backend()
            saved = ctx.saved_tensors
            xs, ys = saved[:ctx.k1], saved[ctx.k1:]
            gs = [g.contiguous() for g in gs]
            xgs = [torch.zeros_like(t) for t in xs]
            ygs = [torch.zeros_like(t) for t in ys]
            for xi, yi, ri, offs in ctx.triples:
                G = gb.SO3part.view(gs[ri])
                getattr(gb.SO3part.view(xgs[xi]), "add_%s_back0" % name)(G, gb.SO3part.view(ys[yi]), offs)
                getattr(gb.SO3part.view(ygs[yi]), "add_%s_back1" % name)(G, gb.SO3part.view(xs[xi]), offs)
            return tuple([None, None, None] + xgs + ygs)

    Fn.__name__ = "O3vec_%sFn" % name
    return Fn


O3vec_CGproductFn = _vec_fn(False)
O3vec_DiagCGproductFn = _vec_fn(True)


class O3vec:
    """{mu: (b, 2l+1, n_mu) tensor}, mu = (l, p) (python/src/gelib/O3vec.py:20-120)."""

    def __init__(self, parts=None):
        self.parts = {}
        for mu, t in (parts or {}).items():
            _check_mu(mu)
            self.parts[mu] = t

    @classmethod
    def zeros(cls, b, tau, device='cpu'):
        return O3vec({mu: torch.zeros([b, 2 * mu[0] + 1, n], dtype=torch.complex64, device=device) for mu, n in tau.items()})

    @classmethod
    def randn(cls, b, tau, device='cpu'):
        return O3vec({mu: torch.randn([b, 2 * mu[0] + 1, n], dtype=torch.complex64, device=device) for mu, n in tau.items()})

    @classmethod
    def zeros_like(cls, x):
        return O3vec({mu: torch.zeros_like(p) for mu, p in x.parts.items()})

    @classmethod
    def randn_like(cls, x):
        return O3vec({mu: torch.randn_like(p) for mu, p in x.parts.items()})

    def getb(self):
        return next(iter(self.parts.values())).size(0)

    def tau(self):
        return O3type({mu: p.size(-1) for mu, p in self.parts.items()})

    get_type = tau

    def requires_grad_(self):
        for p in self.parts.values():
            p.requires_grad_()

    def get_grad(self):
        return O3vec({mu: p.grad for mu, p in self.parts.items()})

    def apply(self, R):
        return O3vec({mu: _plain(O3part(p, mu).apply(R)) for mu, p in self.parts.items()})

    def odot(self, y):
        assert list(self.parts) == list(y.parts)
        return sum(torch.sum(torch.view_as_real(self.parts[mu]) * torch.view_as_real(y.parts[mu])) for mu in self.parts)

    def __add__(self, y):
        assert list(self.parts) == list(y.parts)
        return O3vec({mu: self.parts[mu] + y.parts[mu] for mu in self.parts})

    def _product(self, y, maxl, fn):
        assert isinstance(y, O3vec)
        xmus = sorted(self.parts, key=_index)
        ymus = sorted(y.parts, key=_index)
        args = [self.parts[mu] for mu in xmus] + [y.parts[mu] for mu in ymus]
        rs = fn.apply(tuple(xmus), tuple(ymus), -1 if maxl is None else maxl, *args)
        tau = getattr(self.tau(), "DiagCGproduct" if fn is O3vec_DiagCGproductFn else "CGproduct")(y.tau(), -1 if maxl is None else maxl)
        return O3vec(dict(zip(tau, rs)))

    def CGproduct(self, y, maxl=-1):
        return self._product(y, maxl, O3vec_CGproductFn)

    def DiagCGproduct(self, y, maxl=-1):
        return self._product(y, maxl, O3vec_DiagCGproductFn)

    def __repr__(self):
        return "<O3vec of type %s [b=%d]>" % (dict(self.tau()), self.getb())
