"""Helpers shared by the SO3part / SO3vec classes (python/src/gelib/gelib_common.py:15-20 in the reference)."""


def common_batch(x, y):
    assert x.dim() >= 1
    assert y.dim() >= 1
    if x.size(0) > 1 and y.size(0) > 1:
        assert x.size(0) == y.size(0)
    return max(x.size(0), y.size(0))


def backend():
    """The compiled extension; importing it fails loudly if it has not been built."""
    from gelib_amd import gelib_base
    return gelib_base
