"""The grid ("Arr") variants of the Python surface on the GPU: gelib_amd.SO3partArr / SO3vecArr.  The identities of
the reference's CI suite (python/tests/ci_tests/test_SO3partArr.py, test_SO3vecArr.py: equivariance under a random
rotation, exact bilinearity of the gradients, batch-broadcast operands), agreement with the CPU oracle on the
collapsed cells, and the strided-view case of python/tests/bug1.py."""
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


@pytest.mark.parametrize("b", [1, 2])
@pytest.mark.parametrize("l", [1, 2, 4])
@pytest.mark.parametrize("n", [1, 4, 8])
@pytest.mark.parametrize("diag", [False, True])
def test_part_equivariance(G, b, l, n, diag):
    fn = G.DiagCGproduct if diag else G.CGproduct
    x = G.SO3partArr.randn(b, [2, 2], l, n, device="cuda")
    y = G.SO3partArr.randn(b, [2, 2], l, n, device="cuda")
    z = fn(x, y, l)
    assert isinstance(z, G.SO3partArr) and list(z.shape) == [b, 2, 2, 2 * l + 1, n if diag else n * n]
    R = G.SO3element.random()
    zr = fn(x.apply(R), y.apply(R), l)
    assert torch.allclose(z.apply(R), zr, rtol=1e-3, atol=1e-4)


def part_backprop(G, b, A, l, n, fn, bx=None):
    x = G.SO3partArr.randn(bx or b, A, l, n, device="cuda")
    y = G.SO3partArr.randn(b, A, l, n, device="cuda")
    x.requires_grad_()
    y.requires_grad_()
    z = fn(x, y, l)
    test_vec = G.SO3partArr.randn_like(z)
    loss = z.odot(test_vec)
    loss.backward(torch.tensor(1.0, device="cuda"))
    xeps = G.SO3partArr.randn_like(x)
    xloss = fn(x + xeps, y, l).odot(test_vec)
    assert torch.allclose(xloss - loss, xeps.odot(x.grad), rtol=1e-3, atol=1e-3)
    yeps = G.SO3partArr.randn_like(y)
    yloss = fn(x, y + yeps, l).odot(test_vec)
    assert torch.allclose(yloss - loss, yeps.odot(y.grad), rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("b", [1, 2])
@pytest.mark.parametrize("l", [1, 2, 4])
@pytest.mark.parametrize("n", [1, 4, 8])
@pytest.mark.parametrize("diag", [False, True])
def test_part_backprop(G, b, l, n, diag):
    part_backprop(G, b, [2, 2], l, n, G.DiagCGproduct if diag else G.CGproduct)


@pytest.mark.parametrize("b", [1, 2])
@pytest.mark.parametrize("l", [2, 4])
def test_part_backprop_bcast(G, b, l):
    part_backprop(G, b, [2, 2], l, 4, G.CGproduct, bx=1)


def test_part_matches_oracle(G):
    b, A, l1, l2, l, n1, n2 = 3, [2, 5], 2, 3, 4, 4, 8
    x = G.SO3partArr.randn(b, A, l1, n1, device="cuda")
    y = G.SO3partArr.randn(b, A, l2, n2, device="cuda")
    z = G.CGproduct(x, y, l)
    hx = U.host(x).reshape(-1, 2 * l1 + 1, n1)
    hy = U.host(y).reshape(-1, 2 * l2 + 1, n2)
    want = ora.cg_fwd(hx, hy, l)
    assert U.gate_excess(U.host(z).reshape(want.shape), want) <= 1.0


@pytest.mark.parametrize("maxl", [2, 4])
@pytest.mark.parametrize("nc", [1, 4])
@pytest.mark.parametrize("b", [1, 3])
@pytest.mark.parametrize("diag", [False, True])
def test_vec_equivariance(G, b, nc, maxl, diag):
    fn = G.DiagCGproduct if diag else G.CGproduct
    tau = {l: nc for l in range(maxl + 1)}
    x = G.SO3vecArr.randn(b, [2, 2], tau, device="cuda")
    y = G.SO3vecArr.randn(b, [2, 2], tau, device="cuda")
    R = G.SO3element.random()
    z = fn(x, y, maxl=maxl)
    zr = fn(x.apply(R), y.apply(R), maxl=maxl)
    rz = z.apply(R)
    for i in range(maxl + 1):
        assert list(z.parts[i].shape[:3]) == [b, 2, 2]
        assert torch.allclose(rz.parts[i], zr.parts[i], rtol=1e-3, atol=1e-4)


@pytest.mark.parametrize("nc", [1, 4])
@pytest.mark.parametrize("maxl", [2, 4])
@pytest.mark.parametrize("b", [1, 3])
@pytest.mark.parametrize("diag", [False, True])
@pytest.mark.parametrize("bcast", [False, True])
def test_vec_backprop(G, b, nc, maxl, diag, bcast):
    fn = G.DiagCGproduct if diag else G.CGproduct
    tau = {l: nc for l in range(maxl + 1)}
    x = G.SO3vecArr.randn(1 if bcast else b, [2, 2], tau, device="cuda")
    y = G.SO3vecArr.randn(b, [2, 2], tau, device="cuda")
    x.requires_grad_()
    y.requires_grad_()
    z = fn(x, y)
    test_vec = G.SO3vecArr.randn_like(z)
    loss = z.odot(test_vec)
    loss.backward(torch.tensor(1.0, device="cuda"))
    xgrad, ygrad = x.get_grad(), y.get_grad()
    xeps = G.SO3vecArr.randn_like(x)
    xloss = fn(x + xeps, y).odot(test_vec)
    assert torch.allclose(xloss - loss, xeps.odot(xgrad), rtol=1e-3, atol=1e-3)
    yeps = G.SO3vecArr.randn_like(y)
    yloss = fn(x, y + yeps).odot(test_vec)
    assert torch.allclose(yloss - loss, yeps.odot(ygrad), rtol=1e-3, atol=1e-3)


def test_vec_matches_oracle_and_uses_fused_kernels(G):
    from gelib_amd import cabi
    tau = {l: 4 for l in range(4)}
    x = G.SO3vecArr.randn(3, [2, 3], tau, device="cuda")
    y = G.SO3vecArr.randn(3, [2, 3], tau, device="cuda")
    x.requires_grad_()
    y.requires_grad_()
    z = G.CGproduct(x, y, maxl=3)
    assert cabi.last_path() == 2                      # the grid collapses into the cell index of the fused kernels
    flat = lambda v: [U.host(p).reshape(-1, p.shape[-2], p.shape[-1]) for p in v.parts.values()]
    hx, hy = flat(x), flat(y)
    want = ora.vec_fwd(hx, hy, 3)
    for a, b in zip(flat(z), want):
        assert U.gate_excess(a, b) <= 1.0
    g = [torch.randn_like(p) for p in z.parts.values()]
    torch.autograd.backward(list(z.parts.values()), g)
    assert cabi.last_path() == 2
    hg = [U.host(t).reshape(-1, t.shape[-2], t.shape[-1]) for t in g]
    O = U.VecOracle(hx, hy, 3, False, gs=hg)
    O.check_bwd(flat(x.get_grad()), flat(y.get_grad()), "grid vec grad")


def test_strided_views(G):
    # python/tests/bug1.py: parts that are permuted views of other tensors (no stride is the packed one)
    gen = torch.Generator().manual_seed(5)

    def strided(shape_tail):
        t = torch.randn((1, 2, 3) + shape_tail + (2,), generator=gen)
        t = torch.view_as_complex(t.contiguous())
        t = t.permute((-3, -2, -1, 0, 1))
        t = torch.stack([t[0], t[1], t[1], t[2], t[2]], dim=0)
        return t.permute((3, 4, 0, 1, 2))

    def as_strided_on_gpu(t):
        # same values and the same (non-packed) strides on the device
        d = torch.empty_strided(t.shape, t.stride(), dtype=t.dtype, device="cuda")
        d.copy_(t)
        return d

    a = strided((1, 2))   # (1, 2, 5, 1, 2): l = 0, n = 2
    b = strided((3, 4))   # (1, 2, 5, 3, 4): l = 1, n = 4
    a, b = as_strided_on_gpu(a), as_strided_on_gpu(b)
    assert not a.is_contiguous() and not b.is_contiguous()
    c, d = torch.randn_like(a.contiguous()), torch.randn_like(b.contiguous())
    p1, p3 = G.SO3partArr(a), G.SO3partArr(c)
    z = p1.CGproduct(p3, 0)
    want = ora.cg_fwd(U.host(a.contiguous()).reshape(-1, 1, 2), U.host(c).reshape(-1, 1, 2), 0)
    assert U.gate_excess(U.host(z).reshape(want.shape), want) <= 1.0
    arr1 = G.SO3vecArr(G.SO3partArr(a), G.SO3partArr(b))
    arr2 = G.SO3vecArr(G.SO3partArr(c), G.SO3partArr(d))
    w = arr1.CGproduct(arr2)
    flat = lambda L: [U.host(t.contiguous()).reshape(-1, t.shape[-2], t.shape[-1]) for t in L]
    want = ora.vec_fwd(flat([a, b]), flat([c, d]))
    for got, ref in zip(flat(list(w.parts.values())), want):
        assert U.gate_excess(got, ref) <= 1.0
