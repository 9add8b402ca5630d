"""The O(3) wrappers on the GPU: gelib_amd.O3part / O3vec.  The identities the reference's suite holds for SO(3)
(python/tests/ci_tests/test_SO3part.py, test_SO3vec.py), here under O(3) elements of both determinants, plus
agreement with the CPU oracle: an O(3) product is the SO(3) product of the same tensors, block by block, at the
running channel offset of each output part."""
import numpy as np
import pytest

from oracle import cg_oracle as ora
from tests import gpu_util as U

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def G():
    assert torch.cuda.is_available()
    import gelib_amd
    from gelib_amd import gelib_base  # noqa: F401  (fails loudly if the extension was not built)
    return gelib_amd


def elements(G):
    R = G.O3element.random()
    if R.parity() < 0:
        R = G.O3element(-R)
    return [R, G.O3element(-R), G.O3element(torch.diag(torch.tensor([1.0, 1.0, -1.0])))]   # rotation, improper, mirror


@pytest.mark.parametrize("p1,p2", [(1, 1), (1, -1), (-1, -1)])
@pytest.mark.parametrize("l1,l2,l", [(1, 1, 1), (2, 1, 2), (2, 3, 4)])
@pytest.mark.parametrize("diag", [False, True])
def test_part_equivariance(G, p1, p2, l1, l2, l, diag):
    name = "DiagCGproduct" if diag else "CGproduct"
    x = G.O3part.randn(2, (l1, p1), 4, device="cuda")
    y = G.O3part.randn(2, (l2, p2), 4, device="cuda")
    mu = (l, p1 * p2)
    z = getattr(x, name)(y, mu)
    assert isinstance(z, G.O3part) and z.mu == mu and list(z.shape) == [2, 2 * l + 1, 4 if diag else 16]
    want = ora.cg_fwd(U.host(x), U.host(y), l, diag=diag)
    assert U.gate_excess(U.host(z), want) <= 1.0
    for R in elements(G):
        zr = getattr(x.apply(R), name)(y.apply(R), mu)
        assert torch.allclose(z.apply(R), zr, rtol=1e-3, atol=1e-4)
    with pytest.raises(AssertionError):
        getattr(x, name)(y, (l, -p1 * p2))


def test_part_backprop(G):
    x = G.O3part.randn(3, (2, -1), 4, device="cuda")
    y = G.O3part.randn(3, (1, -1), 4, device="cuda")
    x.requires_grad_()
    y.requires_grad_()
    z = x.CGproduct(y, (2, 1))
    t = G.O3part.randn_like(z)
    loss = z.odot(t)
    loss.backward(torch.tensor(1.0, device="cuda"))
    xeps = G.O3part.randn_like(x)
    assert torch.allclose(G.O3part(x + xeps, x.mu).CGproduct(y, (2, 1)).odot(t) - loss, xeps.odot(x.grad), rtol=1e-3,
                          atol=1e-3)
    yeps = G.O3part.randn_like(y)
    assert torch.allclose(x.CGproduct(G.O3part(y + yeps, y.mu), (2, 1)).odot(t) - loss, yeps.odot(y.grad), rtol=1e-3,
                          atol=1e-3)


TAUS = [({(0, 1): 2, (1, -1): 2, (2, 1): 2}, {(0, 1): 2, (1, -1): 2, (2, 1): 2}),
        ({(0, 1): 3, (1, 1): 3, (1, -1): 3}, {(1, -1): 3, (2, -1): 3})]


def oracle_vec(x, y, diag, maxl):
    """Block by block with the part-level oracle, in the order of O3/O3index.hpp:28-31 and core/Gvec.hpp:311-321."""
    idx = lambda mu: 2 * mu[0] + (mu[1] == -1)
    xm, ym = sorted(x, key=idx), sorted(y, key=idx)
    sizes = {}
    for a in xm:
        for b in ym:
            for l in range(abs(a[0] - b[0]), a[0] + b[0] + 1):
                if maxl >= 0 and l > maxl:
                    continue
                mu = (l, a[1] * b[1])
                sizes[mu] = sizes.get(mu, 0) + (x[a].shape[2] if diag else x[a].shape[2] * y[b].shape[2])
    B = next(iter(x.values())).shape[0]
    out = {mu: np.zeros((B, 2 * mu[0] + 1, n), np.complex64) for mu, n in sizes.items()}
    offs = {mu: 0 for mu in sizes}
    for a in xm:
        for b in ym:
            for l in range(abs(a[0] - b[0]), a[0] + b[0] + 1):
                mu = (l, a[1] * b[1])
                if mu not in out:
                    continue
                ora.part_op(ora.DIAG_FWD if diag else ora.CG_FWD, out[mu], x[a], y[b], offs[mu])
                offs[mu] += x[a].shape[2] if diag else x[a].shape[2] * y[b].shape[2]
    return out


@pytest.mark.parametrize("case", [0, 1])
@pytest.mark.parametrize("diag", [False, True])
@pytest.mark.parametrize("maxl", [-1, 2])
def test_vec_product(G, case, diag, maxl):
    name = "DiagCGproduct" if diag else "CGproduct"
    taux, tauy = (G.O3type(t) for t in TAUS[case])
    x = G.O3vec.randn(3, taux, device="cuda")
    y = G.O3vec.randn(3, tauy, device="cuda")
    z = getattr(x, name)(y, maxl)
    assert dict(z.tau()) == dict(getattr(taux, name)(tauy, maxl))
    want = oracle_vec({mu: U.host(p) for mu, p in x.parts.items()}, {mu: U.host(p) for mu, p in y.parts.items()}, diag,
                      maxl)
    assert set(want) == set(z.parts)
    for mu in want:
        assert U.gate_excess(U.host(z.parts[mu]), want[mu]) <= 1.0, mu
    for R in elements(G):
        zr = getattr(x.apply(R), name)(y.apply(R), maxl)
        rz = z.apply(R)
        for mu in z.parts:
            assert torch.allclose(rz.parts[mu], zr.parts[mu], rtol=1e-3, atol=1e-4), mu


@pytest.mark.parametrize("diag", [False, True])
def test_vec_backprop(G, diag):
    fn = G.DiagCGproduct if diag else G.CGproduct
    taux, tauy = (G.O3type(t) for t in TAUS[1])
    x = G.O3vec.randn(2, taux, device="cuda")
    y = G.O3vec.randn(2, tauy, device="cuda")
    x.requires_grad_()
    y.requires_grad_()
    z = fn(x, y)
    t = G.O3vec.randn_like(z)
    loss = z.odot(t)
    loss.backward(torch.tensor(1.0, device="cuda"))
    xeps = G.O3vec.randn_like(x)
    assert torch.allclose(fn(x + xeps, y).odot(t) - loss, xeps.odot(x.get_grad()), rtol=1e-3, atol=1e-3)
    yeps = G.O3vec.randn_like(y)
    assert torch.allclose(fn(x, y + yeps).odot(t) - loss, yeps.odot(y.get_grad()), rtol=1e-3, atol=1e-3)
