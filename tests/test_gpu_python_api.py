"""The Python surface (gelib_amd.SO3part / SO3vec / CGproduct / DiagCGproduct with autograd) on the GPU: the
identities of the reference's own CI suite (python/tests/ci_tests/test_SO3part.py, test_SO3vec.py) --
equivariance under a random rotation and exact bilinearity of the gradients -- plus agreement with the CPU oracle."""
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


def part_part_backprop(G, b, l, n, fn, arg0, bx=None):
    x = G.SO3part.randn(bx or b, l, n, device="cuda")
    y = G.SO3part.randn(b, l, n, device="cuda")
    x.requires_grad_()
    y.requires_grad_()
    z = fn(x, y, arg0)
    test_vec = G.SO3part.randn_like(z)
    loss = z.odot(test_vec)
    loss.backward(torch.tensor(1.0, device="cuda"))
    xeps = G.SO3part.randn_like(x)
    xloss = fn(x + xeps, y, arg0).odot(test_vec)
    assert torch.allclose(xloss - loss, xeps.odot(x.grad), rtol=1e-3, atol=1e-3)
    yeps = G.SO3part.randn_like(y)
    yloss = fn(x, y + yeps, arg0).odot(test_vec)
    assert torch.allclose(yloss - loss, yeps.odot(y.grad), rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("b", [1, 2])
@pytest.mark.parametrize("l", [1, 2, 4])
@pytest.mark.parametrize("n", [1, 2, 4, 8])
@pytest.mark.parametrize("diag", [False, True])
def test_part_equivariance(G, b, l, n, diag):
    fn = G.DiagCGproduct if diag else G.CGproduct
    x = G.SO3part.randn(b, l, n, device="cuda")
    y = G.SO3part.randn(b, l, n, device="cuda")
    z = fn(x, y, l)
    R = G.SO3element.random()
    zr = fn(x.apply(R), y.apply(R), l)
    assert torch.allclose(z.apply(R), zr, rtol=1e-3, atol=1e-4)


@pytest.mark.parametrize("b", [1, 2])
@pytest.mark.parametrize("l", [1, 2, 4])
@pytest.mark.parametrize("n", [1, 4, 8])
@pytest.mark.parametrize("diag", [False, True])
def test_part_backprop(G, b, l, n, diag):
    part_part_backprop(G, b, l, n, G.DiagCGproduct if diag else G.CGproduct, l)


@pytest.mark.parametrize("b", [2, 5])
@pytest.mark.parametrize("l", [2, 4])
def test_part_backprop_bcast(G, b, l):
    part_part_backprop(G, b, l, 4, G.CGproduct, l, bx=1)


def test_part_matches_oracle(G):
    x = G.SO3part.randn(4, 2, 8, device="cuda")
    y = G.SO3part.randn(4, 3, 8, device="cuda")
    z = G.CGproduct(x, y, 4)
    assert isinstance(z, G.SO3part) and z.shape == (4, 9, 64) and z.dtype == torch.complex64
    assert U.gate_excess(U.host(z), ora.cg_fwd(U.host(x), U.host(y), 4)) <= 1.0
    zd = G.DiagCGproduct(x, x, 3)
    assert U.gate_excess(U.host(zd), ora.cg_fwd(U.host(x), U.host(x), 3, diag=True)) <= 1.0


@pytest.mark.parametrize("maxl", [2, 4])
@pytest.mark.parametrize("b", [1, 3])
@pytest.mark.parametrize("nc", [1, 4])
@pytest.mark.parametrize("diag", [False, True])
def test_vec_equivariance(G, b, nc, maxl, diag):
    fn = G.DiagCGproduct if diag else G.CGproduct
    tau = {l: nc for l in range(maxl + 1)}
    x = G.SO3vec.randn(b, tau, device="cuda")
    y = G.SO3vec.randn(b, tau, device="cuda")
    R = G.SO3element.random()
    z = fn(x, y, maxl=maxl)
    zr = fn(x.apply(R), y.apply(R), maxl=maxl)
    rz = z.apply(R)
    for i in range(maxl + 1):
        assert torch.allclose(rz.parts[i], zr.parts[i], rtol=1e-3, atol=1e-4)


@pytest.mark.parametrize("nc", [1, 4])
@pytest.mark.parametrize("maxl", [2, 4])
@pytest.mark.parametrize("b", [1, 3])
@pytest.mark.parametrize("diag", [False, True])
@pytest.mark.parametrize("bcast", [False, True])
def test_vec_backprop(G, b, nc, maxl, diag, bcast):
    fn = G.DiagCGproduct if diag else G.CGproduct
    tau = {l: nc for l in range(maxl + 1)}
    x = G.SO3vec.randn(1 if bcast else b, tau, device="cuda")
    y = G.SO3vec.randn(b, tau, device="cuda")
    x.requires_grad_()
    y.requires_grad_()
    z = fn(x, y)
    test_vec = G.SO3vec.randn_like(z)
    loss = z.odot(test_vec)
    loss.backward(torch.tensor(1.0, device="cuda"))
    xgrad, ygrad = x.get_grad(), y.get_grad()
    xeps = G.SO3vec.randn_like(x)
    xloss = fn(x + xeps, y).odot(test_vec)
    assert torch.allclose(xloss - loss, xeps.odot(xgrad), rtol=1e-3, atol=1e-3)
    yeps = G.SO3vec.randn_like(y)
    yloss = fn(x, y + yeps).odot(test_vec)
    assert torch.allclose(yloss - loss, yeps.odot(ygrad), rtol=1e-3, atol=1e-3)


def test_vec_matches_oracle_and_uses_fused_kernels(G):
    from gelib_amd import cabi
    tau = {l: 16 for l in range(5)}
    x = G.SO3vec.randn(7, tau, device="cuda")
    y = G.SO3vec.randn(7, tau, device="cuda")
    x.requires_grad_()
    y.requires_grad_()
    z = G.CGproduct(x, y, maxl=4)
    assert cabi.last_path() == 2
    assert {l: p.size(-1) for l, p in z.parts.items()} == {0: 1280, 1: 3072, 2: 4096, 3: 4352, 4: 3840}
    hx = [U.host(p) for p in x.parts.values()]
    hy = [U.host(p) for p in y.parts.values()]
    want = ora.vec_fwd(hx, hy, 4)
    for a, b in zip(z.parts.values(), want):
        assert U.gate_excess(U.host(a), b) <= 1.0
    g = [torch.randn_like(p) for p in z.parts.values()]
    torch.autograd.backward(list(z.parts.values()), g)
    assert cabi.last_path() == 2
    hg = [U.host(t) for t in g]
    O = U.VecOracle(hx, hy, 4, False, gs=hg)
    O.check_bwd([U.host(p.grad) for p in x.parts.values()], [U.host(p.grad) for p in y.parts.values()], "vec grad")


def test_errors_are_exceptions(G):
    x = G.SO3part.randn(2, 1, 4)          # host tensor
    with pytest.raises(RuntimeError):
        G.CGproduct(x, x, 1)
    xc = G.SO3part.randn(2, 1, 4, device="cuda")
    with pytest.raises(RuntimeError):
        G.CGproduct(xc, xc, 3)            # l outside the triangle
    with pytest.raises((RuntimeError, AssertionError)):
        G.DiagCGproduct(xc, G.SO3part.randn(2, 1, 5, device="cuda"), 1)
    with pytest.raises((RuntimeError, AssertionError)):
        G.CGproduct(G.SO3part.randn(3, 1, 4, device="cuda"), xc, 1)


def test_product_then_linear_layer(G):
    """CGproduct followed by the channel-mixing layer (SO3vec * SO3weights), gradients through both: the loss is
    linear in the weights and bilinear in (x, y), so finite differences are exact up to rounding."""
    tau = G.SO3type({l: 4 for l in range(3)})
    x = G.SO3vec.randn(5, tau, device="cuda")
    y = G.SO3vec.randn(5, tau, device="cuda")
    x.requires_grad_()
    tau_mid = tau.CGproduct(tau, 2)
    tau_out = G.SO3type({l: 3 for l in range(3)})
    W = G.SO3weights.randn(tau_mid, tau_out, device="cuda").requires_grad_()

    def net(x, y, W):
        return G.CGproduct(x, y, maxl=2) * W

    out = net(x, y, W)
    assert out.tau() == dict(tau_out)
    test_vec = G.SO3vec.randn_like(out)
    loss = out.odot(test_vec)
    loss.backward(torch.tensor(1.0, device="cuda"))
    Weps = G.SO3weights(*[torch.randn_like(w) for w in W.parts])
    W2 = G.SO3weights(*[w.detach() + e for w, e in zip(W.parts, Weps.parts)])
    dW = sum(torch.sum(torch.view_as_real(e) * torch.view_as_real(w.grad)) for e, w in zip(Weps.parts, W.parts))
    assert torch.allclose(net(x, y, W2).odot(test_vec) - loss, dW, rtol=1e-3, atol=1e-2)
    xeps = G.SO3vec.randn_like(x)
    assert torch.allclose(net(x + xeps, y, W).odot(test_vec) - loss, xeps.odot(x.get_grad()), rtol=1e-3, atol=1e-2)


def test_linear_layer_runs_on_the_library_kernel_and_matches_matmul(G):
    """SO3vec * SO3weights on the GPU: values and both gradients against torch.matmul in complex128."""
    from gelib_amd import cabi
    tau_in = G.SO3type({0: 24, 1: 40, 2: 256})
    tau_out = G.SO3type({0: 16, 1: 5, 2: 48})
    x = G.SO3vec.randn(37, tau_in, device="cuda")
    W = G.SO3weights.randn(tau_in, tau_out, device="cuda").requires_grad_()
    x.requires_grad_()
    out = x * W
    assert cabi.last_path() == 1        # the library ran, not torch.matmul
    g = G.SO3vec.randn_like(out)
    out.odot(g).backward()
    for l, w in zip(tau_in, W.parts):
        xp = x.parts[l].detach().as_subclass(torch.Tensor)
        x64 = xp.to(torch.complex128).requires_grad_()
        w64 = w.detach().to(torch.complex128).requires_grad_()
        ref = torch.matmul(x64, w64)
        assert torch.allclose(out.parts[l].detach().as_subclass(torch.Tensor).to(torch.complex128), ref.detach(), rtol=1e-4, atol=1e-3)
        gl = g.parts[l].detach().as_subclass(torch.Tensor).to(torch.complex128)
        # the same scalar as odot: sum of re*re + im*im
        (torch.view_as_real(ref) * torch.view_as_real(gl)).sum().backward()
        assert torch.allclose(x.parts[l].grad.as_subclass(torch.Tensor).to(torch.complex128), x64.grad, rtol=1e-4, atol=1e-3)
        assert torch.allclose(w.grad.to(torch.complex128), w64.grad, rtol=1e-4, atol=2e-3)


@pytest.mark.parametrize("diag", [False, True])
@pytest.mark.parametrize("shared", ["x", "y"])
def test_vec_broadcast_operand_gradients(G, diag, shared):
    """An operand with batch 1 against a batch of 7 (core/Gpart.hpp:168-185): its gradient is the sum over the batch of
    the gradients the same product gives when the operand is repeated 7 times; the other operand's gradient is the
    same in both."""
    B = 7
    tau = {0: 4, 1: 4, 2: 4} if diag else {0: 3, 1: 2, 2: 2}
    fn = G.DiagCGproduct if diag else G.CGproduct
    a1 = G.SO3vec.randn(1, tau, device="cuda")
    bB = G.SO3vec.randn(B, tau, device="cuda")
    aB = G.SO3vec()
    for l, p in a1.parts.items():
        aB.parts[l] = G.SO3part(p.repeat(B, 1, 1).contiguous())
    for v in (a1, bB, aB):
        for p in v.parts.values():
            p.requires_grad_()
    args = (lambda a, b: (a, b)) if shared == "x" else (lambda a, b: (b, a))
    r1 = fn(*args(a1, bB), 3)
    rB = fn(*args(aB, bB), 3)
    ws = [torch.randn_like(torch.view_as_real(p)) for p in r1.parts.values()]
    loss = lambda r: sum((torch.view_as_real(p) * w).sum() for p, w in zip(r.parts.values(), ws))
    for p, q in zip(r1.parts.values(), rB.parts.values()):
        assert torch.equal(torch.view_as_real(p), torch.view_as_real(q))
    g_a1 = torch.autograd.grad(loss(r1), list(a1.parts.values()) + list(bB.parts.values()))
    g_aB = torch.autograd.grad(loss(rB), list(aB.parts.values()) + list(bB.parts.values()))
    k = len(a1.parts)
    for got, rep in zip(g_a1[:k], g_aB[:k]):
        assert got.shape[0] == 1
        assert torch.allclose(got, rep.sum(0, keepdim=True), rtol=1e-4, atol=1e-4)
    for got, rep in zip(g_a1[k:], g_aB[k:]):
        assert torch.allclose(got, rep, rtol=1e-5, atol=1e-5)
    # ... and against the oracle's serial sum over the batch under the parity rules (term sums over the batch too)
    ha = [U.host(p.detach()) for p in a1.parts.values()]
    hb = [U.host(p.detach()) for p in bB.parts.values()]
    hx, hy = args(ha, hb)
    O = U.VecOracle(hx, hy, 3, diag, gs=[U.host(torch.view_as_complex(w.contiguous())) for w in ws])
    got_a, got_b = [U.host(t) for t in g_a1[:k]], [U.host(t) for t in g_a1[k:]]
    got_x, got_y = args(got_a, got_b)
    O.check_bwd(got_x, got_y, "shared %s diag %d" % (shared, diag))


@pytest.mark.parametrize("narrow", ["x", "y"])
def test_vec_product_with_a_one_channel_operand(G, narrow):
    """CGproduct of features with a one-channel vector runs as the DiagCGproduct with the one channel repeated: the same
    product (against the oracle's CGproduct loops) and the same gradients (against the general kernels, called through
    the autograd function directly)."""
    from gelib_amd.SO3vec import SO3vec_CGproductFn
    B = 6
    wide = G.SO3vec.randn(B, {0: 16, 1: 16, 2: 16, 3: 16}, device="cuda")
    thin = G.SO3vec.randn(B, {0: 1, 1: 1, 2: 1}, device="cuda")
    x, y = (thin, wide) if narrow == "x" else (wide, thin)
    for p in list(x.parts.values()) + list(y.parts.values()):
        p.requires_grad_()
    r = G.CGproduct(x, y, 3)
    xp, yp = list(x.parts.values()), list(y.parts.values())
    want = ora.vec_fwd([U.host(p.detach()) for p in xp], [U.host(p.detach()) for p in yp], 3)
    for a, b in zip(r.parts.values(), want):
        assert a.shape == b.shape
        assert U.gate_excess(U.host(a.detach()), b) <= 1.0
    ref = SO3vec_CGproductFn.apply(len(xp), len(yp), 3, *(xp + yp))
    ws = [torch.randn_like(torch.view_as_real(p)) for p in ref]
    loss = lambda parts: sum((torch.view_as_real(p) * w).sum() for p, w in zip(parts, ws))
    g1 = torch.autograd.grad(loss(list(r.parts.values())), xp + yp)
    g2 = torch.autograd.grad(loss(list(ref)), xp + yp)
    for a, b in zip(g1, g2):
        assert a.shape == b.shape
        assert torch.allclose(a, b, rtol=1e-4, atol=1e-4)
