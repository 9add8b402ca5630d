"""gather_map: which slices of a grid dimension are summed into which (python/src/gelib/gather_map.py:16-45).

A map is a list of (source, target) pairs; ``X.gather(gmap, dim)`` returns the array whose slice ``t`` along grid
dimension ``dim`` is the sum of the slices ``s`` of X over the pairs ``(s, t)``.  The pair list lives in the
extension's ``gather_map`` object, which uploads it to the GPU on first use.
"""
import torch

from gelib_amd.gelib_common import backend


class gather_map:

    def __init__(self, x):
        assert isinstance(x, backend().gather_map)
        self.obj = x

    @classmethod
    def sources_targets(cls, sources, targets, n_in=-1, n_out=-1):
        return gather_map(backend().gather_map.sources_targets(list(sources), list(targets), n_in, n_out))

    @classmethod
    def from_matrix(cls, M, n_in, n_out):
        """M: k x 2 integer tensor, one (source, target) pair per row."""
        assert isinstance(M, torch.Tensor)
        assert isinstance(n_in, int)
        assert isinstance(n_out, int)
        return gather_map(backend().gather_map.from_matrix(M.int().cpu(), n_in, n_out))

    @classmethod
    def random(cls, n_in, n_out, p=0.5, seed=0):
        return gather_map(backend().gather_map.random(n_in, n_out, p, seed))

    def inv(self):
        return gather_map(self.obj.inv())

    def d_in(self):
        return self.obj.d_in()

    def d_out(self):
        return self.obj.d_out()

    def pairs(self):
        return self.obj.pairs()

    def __repr__(self):
        return self.obj.__repr__()

    def __str__(self):
        return self.obj.__str__()
