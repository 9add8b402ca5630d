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
