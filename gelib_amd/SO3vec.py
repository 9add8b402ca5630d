"""SO3vec: an SO(3)-covariant vector, a dict {l: (b, 2l+1, n_l) complex64 tensor} -- the class and autograd functions
of python/src/gelib/SO3vec.py:22-309 for the CG product path.  The products are ONE fused launch per call: the
forward writes into uninitialised parts and the backward computes both gradients from a single pass over g."""
import torch

from gelib_amd.SO3weights import mix_channels
from gelib_amd.gelib_common import backend, common_batch
from gelib_amd.SO3part import SO3part


class SO3vec:

    def __init__(self, *args):
        self.parts = {}
        for x in args:
            assert isinstance(x, torch.Tensor)
            p = SO3part(x)
            self.parts[p.getl()] = x

    @classmethod
    def zeros(cls, b, tau, device='cpu'):
        R = SO3vec()
        for l, n in tau.items():
            R.parts[l] = SO3part.zeros(b, l, n, device=device)
        return R

    @classmethod
    def randn(cls, b, tau, device='cpu'):
        R = SO3vec()
        for l, n in tau.items():
            R.parts[l] = SO3part.randn(b, l, n, device=device)
        return R

    @classmethod
    def spharm(cls, l, X):
        """An SO3vec with the single part l holding the spherical harmonics of X (python/src/gelib/SO3vec.py)."""
        R = SO3vec()
        R.parts[l] = SO3part.spharm(l, X)
        return R

    @classmethod
    def zeros_like(cls, x):
        R = SO3vec()
        for l, p in x.parts.items():
            R.parts[l] = SO3part(torch.zeros_like(p))
        return R

    @classmethod
    def randn_like(cls, x):
        R = SO3vec()
        for l, p in x.parts.items():
            R.parts[l] = SO3part.randn_like(p)
        return R

    def backend(self):
        return backend().SO3vec.view(self.parts)

    def getb(self):
        return self.parts[min(self.parts)].size(0)

    def tau(self):
        return {l: p.size(-1) for l, p in self.parts.items()}

    get_type = tau

    def requires_grad_(self):
        for p in self.parts.values():
            p.requires_grad_()

    def get_grad(self):
        return SO3vec(*[p.grad for p in self.parts.values()])

    def apply(self, R):
        r = SO3vec()
        for l, p in self.parts.items():
            r.parts[l] = SO3part(p).apply(R)
        return r

    def odot(self, y):
        assert list(self.parts.keys()) == list(y.parts.keys())
        return sum(SO3part(self.parts[l]).odot(y.parts[l]) for l in self.parts.keys())

    def __add__(self, y):
        assert list(self.parts.keys()) == list(y.parts.keys())
        return SO3vec(*[self.parts[l] + y.parts[l] for l in self.parts.keys()])

    def __mul__(self, y):
        """Multiply every part by the matching weight matrix of an SO3weights (python/src/gelib/SO3vec.py:174-177)."""
        return SO3vec(*[mix_channels(p, w) for p, w in zip(self.parts.values(), y.parts)])

    def CGproduct(self, y, maxl=-1):
        xparts = list(self.parts.values())
        yparts = list(y.parts.values())
        one = _one_channel_side(xparts, yparts)
        if one is not None and (xparts if one == "y" else yparts)[0].size(-1) > 64:
            # features times a one-channel vector (spherical harmonics of one direction per sample, say): block channel
            # i*N2 + j has N2 = 1 (or N1 = 1), so the product is the DiagCGproduct with the one channel repeated.  Up to
            # 64 channels the library runs it that way by itself, forward and backward (every lane reads the one
            # channel, no copy); with more channels its backward pass would fall to the general kernels, so here the
            # channel is repeated by a torch op, whose backward sums the gradient over the channels.
            wide, narrow = (xparts, yparts) if one == "y" else (yparts, xparts)
            n = wide[0].size(-1)
            rep = [p.expand(*p.shape[:-1], n).contiguous() for p in narrow]
            xs, ys = (wide, rep) if one == "y" else (rep, wide)
            return SO3vec(*SO3vec_DiagCGproductFn.apply(len(xs), len(ys), maxl, *(xs + ys)))
        return SO3vec(*SO3vec_CGproductFn.apply(len(xparts), len(yparts), maxl, *(xparts + yparts)))

    def DiagCGproduct(self, y, maxl=-1):
        xparts = list(self.parts.values())
        yparts = list(y.parts.values())
        return SO3vec(*SO3vec_DiagCGproductFn.apply(len(xparts), len(yparts), maxl, *(xparts + yparts)))

    def __repr__(self):
        return "<SO3vec of type %s [b=%d]>" % (self.tau(), self.getb())


def _one_channel_side(xparts, yparts):
    """'y' if every part of y has one channel and the parts of x share one channel count above one (or 'x' the other
    way round), else None."""
    def side(wide, narrow):
        n = wide[0].size(-1)
        return n > 1 and all(p.size(-1) == n for p in wide) and all(p.size(-1) == 1 for p in narrow)
    if side(xparts, yparts):
        return "y"
    if side(yparts, xparts):
        return "x"
    return None


def _product_fn(diag, part_cls=SO3part, prefix="SO3vec"):
    """Autograd function of the fused product; part_cls wraps the output parts.  Works for any number of grid
    dimensions between the batch and the (2l+1, n) tail (the Arr classes use it too)."""
    gb_type = "DiagCGproduct" if diag else "CGproduct"

    class Fn(torch.autograd.Function):

        @staticmethod
        def forward(ctx, k1, k2, maxl, *args):
            gb = backend()
            ctx.k1, ctx.k2 = k1, k2
            ctx.save_for_backward(*args)
            x = gb.SO3vec.view(list(args[0:k1]))
            y = gb.SO3vec.view(list(args[k1:k1 + k2]))
            b = common_batch(args[0], args[k1])
            lead = [b] + list(args[0].shape[1:-2])
            tau = getattr(x.get_tau(), gb_type)(y.get_tau(), maxl)
            # uninitialised outputs: every channel of every part is written exactly once by the fused launch
            rparts = [torch.empty(lead + [2 * l + 1, n], dtype=torch.complex64, device=args[0].device)
                      for l, n in tau.get_parts().items()]
            r = gb.SO3vec.view(rparts)
            (r.setDiagCGproduct if diag else r.setCGproduct)(x, y)
            return tuple(part_cls(t) for t in rparts)

        @staticmethod
        def backward(ctx, *gargs):
            gb = backend()
            k1, k2 = ctx.k1, ctx.k2
            saved = ctx.saved_tensors
            grads = [torch.empty_like(t, memory_format=torch.contiguous_format) for t in saved]
            x = gb.SO3vec.view(list(saved[0:k1]))
            y = gb.SO3vec.view(list(saved[k1:k1 + k2]))
            g = gb.SO3vec.view([t.contiguous() for t in gargs])
            xg = gb.SO3vec.view(grads[0:k1])
            yg = gb.SO3vec.view(grads[k1:k1 + k2])
            lead = gargs[0].shape[:-2]
            if any(t.shape[:-2] != lead for t in saved) and (len(lead) > 3 or any(t.dim() not in (3, len(lead) + 2) for t in saved)):
                # Broadcast operands among more than two grid dimensions: the library sees those fused into one, which
                # an extent of 1 inside them prevents.  The operand enters as a view with stride 0, the fused backward
                # writes one gradient per cell and torch sums them over the cells the operand is shared by.
                wide = [t.expand(*lead, *t.shape[-2:]) for t in saved]
                full = [torch.empty(list(lead) + list(t.shape[-2:]), dtype=t.dtype, device=t.device) if t.shape[:-2] != lead
                        else grads[i] for i, t in enumerate(saved)]
                getattr(gb.SO3vec, "set%s_back" % gb_type)(gb.SO3vec.view(full[0:k1]), gb.SO3vec.view(full[k1:k1 + k2]), g,
                                                           gb.SO3vec.view(wide[0:k1]), gb.SO3vec.view(wide[k1:k1 + k2]))
                grads = [f if f is grads[i] else f.sum_to_size(saved[i].shape) for i, f in enumerate(full)]
            else:
                # a gradient shaped like an operand that is shared by the batch or the grid (extent 1 there) is summed
                # over the cells inside the library, in a fixed order
                getattr(gb.SO3vec, "set%s_back" % gb_type)(xg, yg, g, x, y)
            return tuple([None, None, None] + grads)

    Fn.__name__ = "%s_%sFn" % (prefix, gb_type)
    return Fn


SO3vec_CGproductFn = _product_fn(False)
SO3vec_DiagCGproductFn = _product_fn(True)
