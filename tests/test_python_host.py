"""CPU-side checks of the Python surface: the extension module loads and has the reference's method names, type
arithmetic known answers, Wigner-D helper properties, and host tensors are refused rather than computed elsewhere."""
import pytest

torch = pytest.importorskip("torch")


def test_extension_surface():
    from gelib_amd import gelib_base as gb
    # python/bindings/SO3part_py.cpp:18-44, SO3vec_py.cpp:18-54, SO3type_py.cpp:16-36
    for name in ("view", "add_CGproduct", "add_CGproduct_back0", "add_CGproduct_back1", "add_DiagCGproduct",
                 "add_DiagCGproduct_back0", "add_DiagCGproduct_back1"):
        assert hasattr(gb.SO3part, name), name
    for name in ("view", "get_tau", "addCGproduct", "addCGproduct_back0", "addCGproduct_back1", "addDiagCGproduct",
                 "addDiagCGproduct_back0", "addDiagCGproduct_back1"):
        assert hasattr(gb.SO3vec, name), name
    for name in ("CGproduct", "DiagCGproduct", "get_parts", "maxl"):
        assert hasattr(gb.SO3type, name), name
    assert callable(gb.CGproduct)


def test_type_arithmetic():
    from gelib_amd import gelib_base as gb
    t = gb.SO3type([1, 1, 1])
    assert gb.CGproduct(t, t).get_parts() == {0: 3, 1: 6, 2: 6, 3: 3, 4: 1}
    assert gb.CGproduct(t, t, 2).get_parts() == {0: 3, 1: 6, 2: 6}
    assert gb.SO3type({0: 2, 1: 2}).CGproduct(gb.SO3type({0: 2, 1: 2})).get_parts() == {0: 8, 1: 12, 2: 4}
    assert t.DiagCGproduct(t, 1).get_parts() == {0: 3, 1: 6}
    assert t.maxl() == 2 and len(t) == 3


def test_views_alias_and_describe():
    from gelib_amd import gelib_base as gb
    x = torch.zeros(2, 5, 3, dtype=torch.complex64)
    p = gb.SO3part.view(x)
    assert p.getl() == 2 and p.getn() == 3
    v = gb.SO3vec.view([torch.zeros(2, 3, 4, dtype=torch.complex64), torch.zeros(2, 1, 2, dtype=torch.complex64)])
    assert v.get_tau().get_parts() == {0: 2, 1: 4}
    with pytest.raises(RuntimeError):
        gb.SO3part.view(torch.zeros(2, 4, 3, dtype=torch.complex64))      # even m-dimension
    with pytest.raises(RuntimeError):
        gb.SO3part.view(torch.zeros(2, 5, 3))                               # not complex64


def test_host_tensors_are_refused():
    import gelib_amd as G
    x = G.SO3part.randn(2, 1, 4)
    with pytest.raises(RuntimeError):
        G.CGproduct(x, x, 1)
    u = G.SO3vec.randn(2, {0: 2, 1: 2})
    with pytest.raises(RuntimeError):
        G.CGproduct(u, u)


def test_wigner_helper():
    import gelib_amd as G
    R1, R2 = G.SO3element.random(), G.SO3element.random()
    assert torch.allclose(R1 @ R1.t(), torch.eye(3), atol=1e-5) and torch.det(R1) > 0
    for l in (1, 2, 4):
        rho = G.SO3irrep(l)
        D1, D2, D12 = rho.matrix(R1), rho.matrix(R2), rho.matrix(G.SO3element(R1 @ R2))
        assert torch.allclose(D1 @ D1.conj().t(), torch.eye(2 * l + 1, dtype=torch.complex64), atol=1e-4)
        assert torch.allclose(D1 @ D2, D12, atol=1e-4)      # a representation


def test_arr_surface():
    import gelib_amd as G
    p = G.SO3partArr.randn(2, [3, 4], 2, 5)
    assert (p.getb(), p.get_adims(), p.get_nadims(), p.getl(), p.getn()) == (2, [3, 4], 2, 2, 5)
    assert list(p.zeros_like(1, 7).shape) == [2, 3, 4, 3, 7]
    assert list(p.collapse().shape) == [2, 12, 5, 5]
    v = G.SO3vecArr.zeros(2, [3], {0: 2, 2: 1})
    assert v.tau() == {0: 2, 2: 1} and v.getb() == 2 and v.get_adims() == [3] and v.l_max() == 2
    w = G.SO3vecArr.randn(2, [3], [2, 1])            # tau given as a list: l = 0, 1
    assert w.tau() == {0: 2, 1: 1}
    R = G.SO3element.random()
    assert list(p.apply(R).shape) == list(p.shape)
    with pytest.raises(RuntimeError):
        G.CGproduct(p, p, 2)                          # host tensors are refused, not computed elsewhere
    with pytest.raises(RuntimeError):
        G.CGproduct(v, v)


def test_type_and_weights():
    import gelib_amd as G
    t = G.SO3type({0: 2, 1: 2})
    assert t.CGproduct(t) == {0: 8, 1: 12, 2: 4} and isinstance(t.CGproduct(t), G.SO3type)
    assert G.SO3type({0: 1, 1: 1, 2: 1}).DiagCGproduct(G.SO3type({0: 1, 1: 1, 2: 1}), 1) == {0: 3, 1: 6}
    tau_in, tau_out = G.SO3type({0: 3, 1: 2}), G.SO3type({0: 5, 1: 4})
    W = G.SO3weights.randn(tau_in, tau_out)
    x = G.SO3vec.randn(2, tau_in)
    y = x * W                                        # plain torch matmuls: also defined on the host
    assert y.tau() == {0: 5, 1: 4}
    assert torch.allclose(y.parts[1], torch.matmul(x.parts[1], W.parts[1]))
    lin = G.SO3linear(tau_in, tau_out)
    assert len(list(lin.parameters())) == 2 and lin(x).tau() == {0: 5, 1: 4}
    xa = G.SO3vecArr.randn(2, [3], tau_in)
    assert (xa * W).tau() == {0: 5, 1: 4} and (xa * W).get_adims() == [3]


def test_o3_labels_and_types():
    import gelib_amd as G
    t = G.O3type({(1, 1): 2, (2, -1): 2})
    # (1,+)x(1,+) -> l=0..2 even; (1,+)x(2,-) and (2,-)x(1,+) -> l=1..3 odd; (2,-)x(2,-) -> l=0..4 even
    assert dict(t.CGproduct(t)) == {(0, 1): 8, (1, 1): 8, (1, -1): 8, (2, 1): 8, (2, -1): 8, (3, 1): 4, (3, -1): 8,
                                    (4, 1): 4}
    assert list(t.CGproduct(t)) == sorted(t.CGproduct(t), key=lambda mu: 2 * mu[0] + (mu[1] == -1))
    assert dict(t.DiagCGproduct(t, 1)) == {(0, 1): 4, (1, 1): 4, (1, -1): 4}
    p = G.O3part.randn(2, (2, -1), 3)
    assert (p.getl(), p.getp(), p.getn(), p.getb()) == (2, -1, 3, 2)
    # the representation property, including reflections: D(R1) D(R2) = D(R1 R2)
    R1, R2 = G.O3element.random(), G.O3element(-torch.eye(3))
    for mu in ((1, 1), (1, -1), (3, -1)):
        rho = G.O3irrep(*mu)
        assert torch.allclose(rho.matrix(R1) @ rho.matrix(R2), rho.matrix(G.O3element(R1 @ R2)), atol=1e-4)
    assert torch.allclose(G.O3irrep(2, -1).matrix(R2), -torch.eye(5, dtype=torch.complex64), atol=1e-5)
    with pytest.raises(AssertionError):
        G.O3part.randn(1, (1, 1), 2).CGproduct(G.O3part.randn(1, (1, -1), 2), (2, 1))   # parity rule


def test_gather_map_host_surface():
    import gelib_amd as G
    m = G.gather_map.sources_targets([0, 1, 2, 2], [1, 1, 0, 2])
    assert (m.d_in(), m.d_out()) == (3, 3) and m.pairs() == ([0, 1, 2, 2], [1, 1, 0, 2])
    assert m.inv().pairs() == ([1, 1, 0, 2], [0, 1, 2, 2]) and str(m).splitlines()[1] == "1<-(0,1)"
    # the map of python/tests/test_gather_map.py
    M = torch.tensor([[4, 3, 9, 1], [5, 5, 2, 7]], dtype=torch.int32)
    f = G.gather_map.from_matrix(M.t(), 10, 10)
    assert f.pairs() == ([4, 3, 9, 1], [5, 5, 2, 7]) and (f.d_in(), f.d_out()) == (10, 10)
    r = G.gather_map.random(6, 5, 0.5, seed=1)
    s, t = r.pairs()
    assert 0 < len(s) < 30 and max(s) < 6 and max(t) < 5 and r.pairs() == G.gather_map.random(6, 5, 0.5, seed=1).pairs()
    with pytest.raises(IndexError):
        G.gather_map.sources_targets([0, 7], [0, 0], 3, 3)
    with pytest.raises(Exception):                       # host tensors are refused
        G.SO3partArr.randn(1, [3], 1, 2).gather(m, 0)
