"""SO3weights / SO3linear: the channel-mixing linear layer that consumes a product
(python/src/gelib/SO3weights.py:22-85; SO3vec.__mul__, python/src/gelib/SO3vec.py:174-177).  One complex
(n_in, n_out) matrix per l, applied to the channel index of every part.  The reference does this with torch.matmul; on
the GPU the product of a part with its matrix and the gradient with respect to the part run on the library's
matrix-core kernels for tall, skinny complex matrices (mix_channels below), as does the gradient with respect to the
matrix; tensors on the host stay with torch."""
import torch

from gelib_amd.SO3type import SO3type


class MixChannelsFn(torch.autograd.Function):
    """r = x w over the last index of a contiguous complex64 GPU tensor x, w of shape (n_in, n_out)."""

    @staticmethod
    def forward(ctx, x, w):
        from gelib_amd import cabi
        ctx.save_for_backward(x, w)
        r = torch.empty(x.shape[:-1] + (w.shape[1],), dtype=x.dtype, device=x.device)
        cabi.part_mix_channels(r, x, w)
        return r

    @staticmethod
    def backward(ctx, g):
        from gelib_amd import cabi
        x, w = ctx.saved_tensors
        gx = gw = None
        g = g.contiguous()
        if ctx.needs_input_grad[0]:
            if cabi.mix_channels_ok(g):
                gx = torch.empty_like(x)
                cabi.part_mix_channels(gx, g, w, adjoint=True)
            else:
                gx = torch.matmul(g, w.conj().transpose(0, 1))
        if ctx.needs_input_grad[1]:
            gw = torch.empty_like(w)
            cabi.part_mix_channels_wgrad(gw, x, g)
        return gx, gw


def mix_channels(x, w):
    """torch.matmul(x, w) for a part x (..., n_in) and a matrix w (n_in, n_out): on the GPU through the library's kernel
    when the part is complex64 with an even number of channels, else torch's own matmul."""
    if x.is_cuda and x.dtype == torch.complex64 and w.dtype == torch.complex64 and w.dim() == 2 and x.numel() > 0:
        from gelib_amd import cabi
        xp = x.as_subclass(torch.Tensor).contiguous()
        wp = w.as_subclass(torch.Tensor).contiguous()
        if cabi.mix_channels_ok(xp):
            return MixChannelsFn.apply(xp, wp)
    return torch.matmul(x, w)


class SO3weights:

    def __init__(self, *args):
        self.parts = list(args)

    @classmethod
    def zeros(cls, tau_in, tau_out, device='cpu'):
        assert isinstance(tau_in, SO3type) and isinstance(tau_out, SO3type)
        R = SO3weights()
        for l in tau_in:
            R.parts.append(torch.zeros([tau_in[l], tau_out[l]], dtype=torch.complex64, device=device))
        return R

    @classmethod
    def randn(cls, tau_in, tau_out, device='cpu'):
        assert isinstance(tau_in, SO3type) and isinstance(tau_out, SO3type)
        R = SO3weights()
        for l in tau_in:
            R.parts.append(torch.randn([tau_in[l], tau_out[l]], dtype=torch.complex64, device=device))
        return R

    def requires_grad_(self):
        for w in self.parts:
            w.requires_grad_()
        return self

    def __repr__(self):
        return "<SO3weights " + ",".join("(%d,%d)" % (w.size(0), w.size(1)) for w in self.parts) + ">"


class SO3linear(torch.nn.Module):

    def __init__(self, tau_in, tau_out, device='cpu'):
        super().__init__()
        assert isinstance(tau_in, SO3type) and isinstance(tau_out, SO3type)
        self.W = SO3weights.randn(tau_in, tau_out, device)
        self.weights = torch.nn.ParameterList([torch.nn.Parameter(w) for w in self.W.parts])
        self.W.parts = list(self.weights)

    def forward(self, x):
        return x * self.W


class CGproductLinearFn(torch.autograd.Function):
    """CGproduct(x, y, maxl) * W with the product formed and consumed inside one kernel (forward).  The backward pass
    forms the product again, a chunk of the batch at a time (gelib_hip_so3vec_cg_linear_bwd): the product and its gradient
    exist only for the chunk at hand, in a workspace of at most BWD_WORKSPACE_BYTES, and nothing of the product's size is
    kept between the two passes."""

    BWD_WORKSPACE_BYTES = 8 << 30   # headline type, 32768 cells: 34.6 ms with 1 GiB, 24.5 with 4, 22.0 with 8, 19.5 with 28 (one chunk)

    @staticmethod
    def forward(ctx, k1, k2, maxl, *args):
        from gelib_amd import cabi
        xs, ys, ws = list(args[0:k1]), list(args[k1:k1 + k2]), list(args[k1 + k2:])
        ctx.k1, ctx.k2, ctx.maxl = k1, k2, maxl
        ctx.save_for_backward(*args)
        lead = list(xs[0].shape[:-2])
        out = [torch.empty(lead + [2 * l + 1, w.shape[1]], dtype=torch.complex64, device=xs[0].device)
               for l, w in enumerate(ws)]
        if not cabi.so3vec_cg_linear_fwd(out, xs, ys, ws, accumulate=False):
            raise RuntimeError("CGproduct_linear: shapes outside what the fused kernel takes")
        return tuple(out)

    @staticmethod
    def backward(ctx, *gargs):
        from gelib_amd import cabi
        from gelib_amd.SO3vec import SO3vec
        k1, k2 = ctx.k1, ctx.k2
        saved = ctx.saved_tensors
        xs, ys, ws = list(saved[0:k1]), list(saved[k1:k1 + k2]), list(saved[k1 + k2:])
        need = ctx.needs_input_grad[3:]
        gs = [g.contiguous() for g in gargs]
        xg = [torch.empty_like(t, memory_format=torch.contiguous_format) for t in xs] if any(need[0:k1]) else None
        yg = [torch.empty_like(t, memory_format=torch.contiguous_format) for t in ys] if any(need[k1:k1 + k2]) else None
        wg = [torch.empty_like(t, memory_format=torch.contiguous_format) for t in ws] if any(need[k1 + k2:]) else None
        if cabi.so3vec_cg_linear_bwd(xg, yg, wg, gs, xs, ys, ws, accumulate=False,
                                     workspace_bytes=CGproductLinearFn.BWD_WORKSPACE_BYTES):
            grads = (xg or [None] * k1) + (yg or [None] * k2) + (wg or [None] * len(ws))
            return tuple([None, None, None] + [g if n else None for g, n in zip(grads, need)])
        leaves = [t.detach().requires_grad_() for t in saved]
        with torch.enable_grad():
            x, y = SO3vec(*leaves[0:k1]), SO3vec(*leaves[k1:k1 + k2])
            out = x.CGproduct(y, ctx.maxl) * SO3weights(*leaves[k1 + k2:])
            outs = list(out.parts.values())
        wanted = [t for t, need in zip(leaves, ctx.needs_input_grad[3:]) if need]
        got = iter(torch.autograd.grad(outs, wanted, [g.contiguous() for g in gargs]))
        return tuple([None, None, None] + [next(got) if need else None for need in ctx.needs_input_grad[3:]])


def fused_linear_ok(x, y, W, maxl):
    """True when CGproduct(x, y, maxl) * W is a case of the fused kernel: complex64 parts on one GPU, contiguous, the same
    leading dimensions, l <= 4 and at most 16 channels everywhere, a product with exactly the parts l = 0..4."""
    xs, ys, ws = list(x.parts.values()), list(y.parts.values()), list(W.parts)
    ts = xs + ys + ws
    if not ts or not all(t.is_cuda and t.dtype == torch.complex64 and t.is_contiguous() and t.device == ts[0].device
                         for t in ts):
        return False
    if any(t.shape[:-2] != xs[0].shape[:-2] for t in xs + ys) or xs[0].numel() == 0:
        return False
    if max(x.parts) > 4 or max(y.parts) > 4 or any(t.shape[-1] > 16 for t in xs + ys):
        return False
    from gelib_amd import cabi
    taus = cabi.so3type_product(x.tau(), y.tau(), maxl)
    if sorted(taus) != [0, 1, 2, 3, 4] or len(ws) != 5:
        return False
    return all(w.dim() == 2 and w.shape[0] == taus[l] and 1 <= w.shape[1] <= 16 for l, w in enumerate(ws))


def CGproduct_linear(x, y, W, maxl=-1):
    """x.CGproduct(y, maxl) * W (python/src/gelib/SO3vec.py:174-177 applied to the result of SO3vec.CGproduct).  On the GPU,
    for the shapes fused_linear_ok accepts, one kernel forms the product and multiplies it by the matrices without
    storing it; every other case runs the two steps one after the other."""
    from gelib_amd.SO3vec import SO3vec
    if fused_linear_ok(x, y, W, maxl):
        xs = [p.as_subclass(torch.Tensor) for p in x.parts.values()]
        ys = [p.as_subclass(torch.Tensor) for p in y.parts.values()]
        ws = [w.as_subclass(torch.Tensor) for w in W.parts]
        return SO3vec(*CGproductLinearFn.apply(len(xs), len(ys), maxl, *(xs + ys + ws)))
    return x.CGproduct(y, maxl) * W
