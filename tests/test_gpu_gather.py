"""Sums of slices along a grid dimension (gather) on the GPU, through the C-ABI and through the Python classes.

The reference has no numeric test of gather (python/tests/test_gather_map.py only prints two maps), and the loop it
calls lives in cnine, outside its tree.  What pins the result here is the definition itself: a gather is the product
with the 0/1 incidence matrix of the pairs, computed with torch on the host in float64; the numpy loop of the oracle
adds in the same order as the kernel and must match bit for bit."""
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


def random_pairs(n_in, n_out, k, seed):
    rng = np.random.default_rng(seed)
    return rng.integers(0, n_in, k).tolist(), rng.integers(0, n_out, k).tolist()


def cplx(*shape, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.view_as_complex(torch.randn(*shape, 2, generator=g))


@pytest.mark.parametrize("shape,dim,n_out,k", [
    ((3, 7, 5, 4), 1, 6, 20),          # one grid dimension
    ((2, 5, 6, 3, 8), 1, 9, 30),       # first of two
    ((2, 5, 6, 3, 8), 2, 4, 11),       # second of two
    ((40, 3, 16), 0, 17, 100),         # along the batch
    ((1, 300, 7, 16), 1, 70000, 900),  # more targets than one launch takes rows, most of them empty
    ((2, 4, 1, 1), 1, 4, 0),           # no pairs at all
])
@pytest.mark.parametrize("accumulate", [True, False])
def test_cabi_gather_matches_oracle_bit_for_bit(G, shape, dim, n_out, k, accumulate):
    from gelib_amd import cabi
    x = cplx(*shape, seed=1)
    src, tgt = random_pairs(shape[dim], n_out, k, 2)
    rshape = list(shape)
    rshape[dim] = n_out
    r0 = cplx(*rshape, seed=3)
    gm = cabi.GatherMap(src, tgt, shape[dim], n_out)
    r = r0.cuda()
    cabi.part_gather(r, x.cuda(), gm, dim, accumulate=accumulate)
    want = ora.gather(x.numpy(), src, tgt, n_out, dim, r=r0.numpy().copy() if accumulate else None)
    assert np.array_equal(U.host(r), want)
    # the inverse map: sources and targets change places
    g = cplx(*rshape, seed=4)
    xg = torch.zeros(shape, dtype=torch.complex64, device="cuda")
    cabi.part_gather(xg, g.cuda(), gm, dim, inverse=True)
    assert np.array_equal(U.host(xg), ora.gather(g.numpy(), tgt, src, shape[dim], dim))


def test_cabi_gather_is_the_incidence_matrix_product(G):
    from gelib_amd import cabi
    n_in, n_out = 11, 7
    src, tgt = random_pairs(n_in, n_out, 40, 5)
    A = torch.zeros(n_out, n_in, dtype=torch.float64)
    for s, t in zip(src, tgt):
        A[t, s] += 1                      # a repeated pair counts twice
    x = cplx(3, n_in, 5, 4, seed=6)
    r = torch.zeros(3, n_out, 5, 4, dtype=torch.complex64, device="cuda")
    cabi.part_gather(r, x.cuda(), cabi.GatherMap(src, tgt, n_in, n_out), 1)
    want = torch.einsum("ts,bsmc->btmc", A.to(torch.complex128), x.to(torch.complex128))
    assert torch.allclose(r.cpu().to(torch.complex128), want, rtol=1e-5, atol=1e-5)


def test_cabi_gather_strided_and_errors(G):
    from gelib_amd import cabi
    src, tgt = [0, 2, 2, 1], [1, 1, 0, 3]
    gm = cabi.GatherMap(src, tgt, 3, 4)
    big = cplx(2, 3, 5, 12, seed=7).cuda()
    x = big[..., 2:10:2]                  # channel stride 2
    r = torch.zeros(2, 4, 5, 4, dtype=torch.complex64, device="cuda")
    cabi.part_gather(r, x, gm, 1)
    assert np.array_equal(U.host(r), ora.gather(U.host(x), src, tgt, 4, 1))
    with pytest.raises(cabi.GelibHipError) as e:      # wrong extent along the gathered dimension
        cabi.part_gather(torch.zeros(2, 5, 5, 4, dtype=torch.complex64, device="cuda"), x, gm, 1)
    assert e.value.status == 7
    with pytest.raises(cabi.GelibHipError) as e:      # other dimensions must agree
        cabi.part_gather(torch.zeros(2, 4, 5, 3, dtype=torch.complex64, device="cuda"), x, gm, 1)
    assert e.value.status == 5
    with pytest.raises(cabi.GelibHipError) as e:      # index outside the map's range
        cabi.GatherMap([0, 3], [0, 0], 3, 4)
    assert e.value.status == 12
    with pytest.raises(cabi.GelibHipError) as e:      # host memory
        cabi.part_gather(r.cpu(), x, gm, 1)
    assert e.value.status == 8


def test_python_gather_and_its_gradient(G):
    gmap = G.gather_map.random(5, 4, 0.4, seed=3)
    src, tgt = gmap.pairs()
    x = G.SO3partArr.randn(2, [5, 3], 2, 4, device="cuda")
    x.requires_grad_()
    y = x.gather(gmap, 0)
    assert isinstance(y, G.SO3partArr) and list(y.shape) == [2, 4, 3, 5, 4]
    assert np.array_equal(U.host(y), ora.gather(U.host(x), src, tgt, 4, 1))
    t = G.SO3partArr.randn_like(y)
    y.odot(t).backward()
    # the gradient is the gather of t along the same pairs read backwards
    assert np.array_equal(U.host(x.grad), ora.gather(U.host(t), tgt, src, 5, 1))
    # second grid dimension, on a vector; gather commutes with the product when each target has one source
    perm = G.gather_map.sources_targets([2, 0, 1], [0, 1, 2])
    tau = {0: 2, 1: 2, 2: 2}
    u = G.SO3vecArr.randn(2, [2, 3], tau, device="cuda")
    v = G.SO3vecArr.randn(2, [2, 3], tau, device="cuda")
    a = G.CGproduct(u, v, maxl=2).gather(perm, 1)
    b = G.CGproduct(u.gather(perm, 1), v.gather(perm, 1), maxl=2)
    for l in a.parts:
        assert torch.equal(a.parts[l], b.parts[l])
    R = G.SO3element.random()              # gather commutes with rotations
    w = u.gather(G.gather_map.random(3, 5, 0.5, seed=9), 1)
    wr = u.apply(R).gather(G.gather_map.random(3, 5, 0.5, seed=9), 1)
    for l in w.parts:
        assert torch.allclose(w.apply(R).parts[l], wr.parts[l], rtol=1e-4, atol=1e-5)
