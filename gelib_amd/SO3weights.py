"""SO3weights / SO3linear: the channel-mixing linear layer that consumes a product
(python/src/gelib/SO3weights.py:22-85; SO3vec.__mul__, python/src/gelib/SO3vec.py:174-177).  One complex
(n_in, n_out) matrix per l, applied to the channel index of every part with torch.matmul -- plain library GEMMs,
differentiable by torch itself."""
import torch

from gelib_amd.SO3type import SO3type


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
