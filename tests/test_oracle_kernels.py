"""Pins the oracle's loop nests (part level and vec level) against independent mathematics:
brute-force loops with exact sympy coefficients, a complex128 einsum, closed-form special cases,
adjoint identities, Wigner-D equivariance and the reference's documented type arithmetic."""
import numpy as np
import pytest

from oracle import cg_oracle as ora
from tests import helpers as H

TOL32 = dict(rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("l1,l2,l,n1,n2,diag", [(1, 1, 1, 2, 3, False), (2, 1, 2, 2, 2, False), (1, 2, 3, 3, 3, True),
                                                  (0, 2, 2, 1, 2, False), (2, 2, 0, 2, 2, True)])
def test_fwd_brute_force_sympy(l1, l2, l, n1, n2, diag):
    rng = np.random.default_rng(1)
    x = H.randc(rng, 2, 2 * l1 + 1, n1, dtype=np.complex128)
    y = H.randc(rng, 2, 2 * l2 + 1, n2, dtype=np.complex128)
    want = H.brute_cg(x, y, H.sympy_cg_matrix(l1, l2, l), l, diag)
    got = ora.cg_fwd(x, y, l, diag)
    assert np.allclose(got, want, rtol=1e-6, atol=1e-6)     # float-rounded table inside the oracle
    got32 = ora.cg_fwd(x.astype(np.complex64), y.astype(np.complex64), l, diag)
    assert np.allclose(got32, want, **TOL32)


@pytest.mark.parametrize("l1,l2,l", [(1, 1, 1), (2, 3, 4), (4, 4, 4), (3, 1, 2), (6, 6, 6), (10, 10, 7)])
@pytest.mark.parametrize("diag", [False, True])
def test_fwd_bwd_einsum(l1, l2, l, diag):
    rng = np.random.default_rng(2)
    n1, n2 = (4, 4) if diag else (3, 5)
    B = 3
    x = H.randc(rng, B, 2 * l1 + 1, n1, dtype=np.complex128)
    y = H.randc(rng, B, 2 * l2 + 1, n2, dtype=np.complex128)
    C = H.golden_cg_tables().get((l1, l2, l))
    if C is None:
        C = H.sympy_cg_matrix(l1, l2, l)
    Cf = C.astype(np.float32)            # the oracle stores the table in float32
    want = H.einsum_cg(x, y, Cf, l, diag)
    got = ora.cg_fwd(x, y, l, diag)
    assert np.allclose(got, want, rtol=1e-12, atol=1e-12)
    g = H.randc(rng, *want.shape, dtype=np.complex128)
    wxg, wyg = H.einsum_cg_bwd(g, x, y, Cf, diag)
    xg, yg = ora.cg_bwd(g, x, y, diag)
    assert np.allclose(xg, wxg, rtol=1e-12, atol=1e-12)
    assert np.allclose(yg, wyg, rtol=1e-12, atol=1e-12)
    # float32 loop-order-faithful path stays inside the parity gate of the exact answer
    x32, y32, g32 = (a.astype(np.complex64) for a in (x, y, g))
    assert np.allclose(ora.cg_fwd(x32, y32, l, diag), want, **TOL32)
    xg32, yg32 = ora.cg_bwd(g32, x32, y32, diag)
    assert np.allclose(xg32, wxg, rtol=1e-4, atol=1e-4)
    assert np.allclose(yg32, wyg, rtol=1e-4, atol=1e-4)


def test_channel_order_and_offset():
    # channel index inside a block is n1*N2+n2 and offs shifts the block (SO3/SO3part.hpp:215,219)
    rng = np.random.default_rng(3)
    x = H.randc(rng, 1, 3, 2, dtype=np.complex128)
    y = H.randc(rng, 1, 5, 3, dtype=np.complex128)
    r = np.zeros((1, 5, 10), dtype=np.complex128)
    ora.part_op(ora.CG_FWD, r, x, y, offs=4)
    assert np.all(r[:, :, :4] == 0)
    C = H.sympy_cg_matrix(1, 2, 2)
    for i in range(2):
        for j in range(3):
            single = H.brute_cg(x[:, :, i:i + 1], y[:, :, j:j + 1], C, 2)
            assert np.allclose(r[:, :, 4 + i * 3 + j], single[:, :, 0], atol=1e-6)


def test_accumulates():
    rng = np.random.default_rng(4)
    x = H.randc(rng, 2, 3, 2)
    y = H.randc(rng, 2, 3, 2)
    r0 = H.randc(rng, 2, 3, 4)
    r = r0.copy()
    ora.part_op(ora.CG_FWD, r, x, y)
    assert np.allclose(r - r0, ora.cg_fwd(x, y, 1), atol=1e-5)


def test_special_cases():
    rng = np.random.default_rng(5)
    # l1 = 0: r = x0 * y
    x = H.randc(rng, 2, 1, 1, dtype=np.complex128)
    y = H.randc(rng, 2, 7, 4, dtype=np.complex128)
    assert np.allclose(ora.cg_fwd(x, y, 3), x * y, atol=1e-6)
    # l = 0, l1 = l2: r = sum_m (-1)^(l1-m)/sqrt(2l1+1) x_m y_-m
    l1 = 3
    x = H.randc(rng, 2, 7, 1, dtype=np.complex128)
    y = H.randc(rng, 2, 7, 1, dtype=np.complex128)
    want = sum((-1) ** (l1 - m) / np.sqrt(7) * x[:, m + l1, 0] * y[:, -m + l1, 0] for m in range(-l1, l1 + 1))
    assert np.allclose(ora.cg_fwd(x, y, 0)[:, 0, 0], want, atol=1e-6)
    # stretched component: r[m=l1+l2] = x[l1] y[l2]
    x = H.randc(rng, 1, 5, 1, dtype=np.complex128)
    y = H.randc(rng, 1, 3, 1, dtype=np.complex128)
    r = ora.cg_fwd(x, y, 3)
    assert np.allclose(r[0, 6, 0], x[0, 4, 0] * y[0, 2, 0], atol=1e-6)
    assert np.allclose(r[0, 0, 0], x[0, 0, 0] * y[0, 0, 0], atol=1e-6)


@pytest.mark.parametrize("diag", [False, True])
def test_adjoint_identities(diag):
    # <CG(x,y), g> = <x, back0(g,y)> = <y, back1(g,x)> with the real inner product
    rng = np.random.default_rng(6)
    x = H.randc(rng, 3, 5, 4, dtype=np.complex128)
    y = H.randc(rng, 3, 7, 4, dtype=np.complex128)
    r = ora.cg_fwd(x, y, 4, diag)
    g = H.randc(rng, *r.shape, dtype=np.complex128)
    xg, yg = ora.cg_bwd(g, x, y, diag)
    assert abs(H.odot(r, g) - H.odot(x, xg)) < 1e-9 * abs(H.odot(r, g)) + 1e-9
    assert abs(H.odot(r, g) - H.odot(y, yg)) < 1e-9 * abs(H.odot(r, g)) + 1e-9


@pytest.mark.parametrize("l1,l2,l", [(1, 1, 1), (2, 2, 2), (4, 4, 4), (2, 3, 4), (3, 2, 1)])
@pytest.mark.parametrize("diag", [False, True])
def test_equivariance(l1, l2, l, diag):
    # D^l(R) CG(x,y) = CG(D^l1(R) x, D^l2(R) y)   (python/tests/ci_tests/test_SO3part.py:55-86)
    rng = np.random.default_rng(7)
    ang = (0.7, 1.1, -0.4)
    x = H.randc(rng, 2, 2 * l1 + 1, 3, dtype=np.complex128)
    y = H.randc(rng, 2, 2 * l2 + 1, 3, dtype=np.complex128)
    lhs = H.rotate(ora.cg_fwd(x, y, l, diag), ang)
    rhs = ora.cg_fwd(H.rotate(x, ang), H.rotate(y, ang), l, diag)
    assert np.allclose(lhs, rhs, rtol=1e-6, atol=1e-6)


def test_batch_broadcast():
    rng = np.random.default_rng(8)
    x = H.randc(rng, 1, 3, 2, dtype=np.complex128)
    y = H.randc(rng, 4, 3, 2, dtype=np.complex128)
    r = ora.cg_fwd(x, y, 2)
    rfull = ora.cg_fwd(np.repeat(x, 4, axis=0), y, 2)
    assert np.allclose(r, rfull)
    g = H.randc(rng, *r.shape, dtype=np.complex128)
    xg, yg = ora.cg_bwd(g, x, y)
    xgf, ygf = ora.cg_bwd(g, np.repeat(x, 4, axis=0), y)
    assert np.allclose(xg, xgf.sum(axis=0, keepdims=True))
    assert np.allclose(yg, ygf)


def test_errors():
    z = np.zeros((2, 3, 4), dtype=np.complex64)
    with pytest.raises(ValueError):
        ora.part_op(ora.CG_FWD, np.zeros((2, 9, 16), dtype=np.complex64), z, z)      # l=4 outside 1x1
    with pytest.raises(ValueError):
        ora.part_op(ora.CG_FWD, np.zeros((2, 3, 15), dtype=np.complex64), z, z)      # 16 channels needed
    with pytest.raises(ValueError):
        ora.part_op(ora.DIAG_FWD, np.zeros((2, 3, 4), dtype=np.complex64), z, np.zeros((2, 3, 5), dtype=np.complex64))
    with pytest.raises(ValueError):
        ora.part_op(ora.CG_FWD, np.zeros((3, 3, 16), dtype=np.complex64), z, z)      # batch 3 vs 2


# ---- vec level --------------------------------------------------------------------------------------------------

def test_type_known_answers():
    # python/docs/source/abandoned/SO3type.rst:28-41
    assert ora.type_product({0: 2, 1: 2}, {0: 2, 1: 2}) == {0: 8, 1: 12, 2: 4}
    assert ora.type_product({0: 1, 1: 1, 2: 1}, {0: 1, 1: 1, 2: 1}) == {0: 3, 1: 6, 2: 6, 3: 3, 4: 1}
    assert ora.type_product({0: 1, 1: 1, 2: 1}, {0: 1, 1: 1, 2: 1}, maxl=2) == {0: 3, 1: 6, 2: 6}
    # headline configuration: L=4, 16 channels per part
    tau = {l: 16 for l in range(5)}
    assert ora.type_product(tau, tau, maxl=4) == {0: 1280, 1: 3072, 2: 4096, 3: 4352, 4: 3840}
    full = ora.type_product(tau, tau)
    assert [full[l] for l in range(9)] == [1280, 3072, 4096, 4352, 3840, 2560, 1536, 768, 256]
    tau6 = {l: 64 for l in range(7)}
    d = ora.type_product(tau6, tau6, maxl=6, diag=True)
    assert [d[l] for l in range(7)] == [448, 1152, 1664, 1984, 2112, 2048, 1792]


@pytest.mark.parametrize("diag", [False, True])
@pytest.mark.parametrize("maxl", [-1, 2])
def test_vec_layout_against_part_products(diag, maxl):
    # blocks are laid out in (l1 ascending, l2 ascending) order with per-l running offsets (core/Gvec.hpp:311-321)
    rng = np.random.default_rng(9)
    tx = {0: 2, 1: 3, 2: 2} if not diag else {0: 2, 1: 2, 3: 2}
    ty = {1: 2, 2: 1} if not diag else {0: 2, 2: 2}
    xs = [H.randc(rng, 2, 2 * l + 1, n, dtype=np.complex128) for l, n in tx.items()]
    ys = [H.randc(rng, 2, 2 * l + 1, n, dtype=np.complex128) for l, n in ty.items()]
    rparts = ora.vec_fwd(xs, ys, maxl, diag)
    tau = ora.type_product(tx, ty, maxl, diag)
    assert [(p.shape[1] - 1) // 2 for p in rparts] == sorted(tau)
    off = {l: 0 for l in tau}
    for x in xs:
        for y in ys:
            l1, l2 = (x.shape[1] - 1) // 2, (y.shape[1] - 1) // 2
            for l in range(abs(l1 - l2), l1 + l2 + 1):
                if l not in tau:
                    continue
                C = H.sympy_cg_matrix(l1, l2, l)
                blk = H.einsum_cg(x, y, C, l, diag)
                n = blk.shape[2]
                rp = rparts[sorted(tau).index(l)]
                assert np.allclose(rp[:, :, off[l]:off[l] + n], blk, atol=1e-6)
                off[l] += n
    assert off == tau


def test_diag_is_subset_of_full_product():
    # Diag output = channels n*(N+1) of each block of the full product (python/docs/source/SO3vecB.rst:117-181)
    rng = np.random.default_rng(10)
    N = 3
    xs = [H.randc(rng, 2, 2 * l + 1, N, dtype=np.complex128) for l in range(3)]
    ys = [H.randc(rng, 2, 2 * l + 1, N, dtype=np.complex128) for l in range(3)]
    full = ora.vec_fwd(xs, ys)
    diag = ora.vec_fwd(xs, ys, diag=True)
    for f, d in zip(full, diag):
        nblk = d.shape[2] // N
        assert f.shape[2] == nblk * N * N
        pick = [b * N * N + n * (N + 1) for b in range(nblk) for n in range(N)]
        assert np.allclose(f[:, :, pick], d)


@pytest.mark.parametrize("diag", [False, True])
def test_vec_adjoint_and_autograd_convention(diag):
    rng = np.random.default_rng(11)
    tau = {0: 2, 1: 2, 2: 2}
    xs = [H.randc(rng, 3, 2 * l + 1, n, dtype=np.complex128) for l, n in tau.items()]
    ys = [H.randc(rng, 3, 2 * l + 1, n, dtype=np.complex128) for l, n in tau.items()]
    r = ora.vec_fwd(xs, ys, 2, diag)
    g = [H.randc(rng, *p.shape, dtype=np.complex128) for p in r]
    xg, yg = ora.vec_bwd(g, xs, ys, diag)
    lhs = sum(H.odot(a, b) for a, b in zip(r, g))
    assert abs(lhs - sum(H.odot(a, b) for a, b in zip(xs, xg))) < 1e-9 * abs(lhs)
    assert abs(lhs - sum(H.odot(a, b) for a, b in zip(ys, yg))) < 1e-9 * abs(lhs)
    # exact bilinearity, the reference's own gradient test (python/tests/ci_tests/test_SO3vec.py:7-29)
    eps = [H.randc(rng, *p.shape, dtype=np.complex128) for p in xs]
    r2 = ora.vec_fwd([a + e for a, e in zip(xs, eps)], ys, 2, diag)
    d = sum(H.odot(a, b) for a, b in zip(r2, g)) - lhs
    assert abs(d - sum(H.odot(e, b) for e, b in zip(eps, xg))) < 1e-9 * abs(d) + 1e-9


def test_threads_match_serial():
    rng = np.random.default_rng(12)
    x = H.randc(rng, 37, 5, 4)
    y = H.randc(rng, 37, 7, 4)
    a = ora.cg_fwd(x, y, 4, nthreads=1)
    b = ora.cg_fwd(x, y, 4, nthreads=4)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("diag", [False, True])
def test_term_sums_are_sums_of_term_moduli(diag):
    """The error-analysis aid of the oracle (|C| on the moduli of the operands) against the definition, with sympy's
    coefficients: einsum over |W|, |x|, |y| forward and |W|, |g|, |y| / |x| backward."""
    rng = np.random.default_rng(21)
    l1, l2, l, n1, n2 = 2, 1, 2, 3, (3 if diag else 2)
    x, y = H.randc(rng, 2, 2 * l1 + 1, n1), H.randc(rng, 2, 2 * l2 + 1, n2)
    C = np.abs(H.sympy_cg_matrix(l1, l2, l))
    ax, ay = np.abs(x).astype(np.complex128), np.abs(y).astype(np.complex128)
    want = H.einsum_cg(ax, ay, C, l, diag).real
    got = ora.vec_fwd_term_sums([x], [y], l, diag)   # parts l = |l1-l2| .. maxl = l: the last one is l
    np.testing.assert_allclose(got[-1], want, rtol=1e-6, atol=1e-12)
    part = ora.part_term_sums(ora.DIAG_FWD if diag else ora.CG_FWD, np.zeros_like(got[-1], dtype=np.complex64), x, y)
    np.testing.assert_allclose(part, want, rtol=1e-6, atol=1e-12)
    g = H.randc(rng, *want.shape)
    wx, wy = H.einsum_cg_bwd(np.abs(g).astype(np.complex128), ax, ay, C, diag)
    sx = ora.part_term_sums(ora.DIAG_BACK0 if diag else ora.CG_BACK0, g, x, y)
    sy = ora.part_term_sums(ora.DIAG_BACK1 if diag else ora.CG_BACK1, g, x, y)
    np.testing.assert_allclose(sx, wx.real, rtol=1e-6, atol=1e-12)
    np.testing.assert_allclose(sy, wy.real, rtol=1e-6, atol=1e-12)
    # every term sum bounds the modulus of the element it belongs to, and the switch is off again afterwards
    r = ora.cg_fwd(x, y, l, diag)
    assert np.all(np.abs(r) <= want * (1 + 1e-6) + 1e-6)
    assert np.any(ora.cg_matrix(l1, l2, l) < 0)


def test_parity_rules_accept_and_reject():
    """Host logic of the per-component parity check (tests/gpu_util.py): rule A, rule B, rule C and a rejection."""
    from tests import gpu_util as U
    e = np.array([100.0 + 0j, 0.001 + 0j, 0.001 + 0j, 0.001 + 0j], dtype=np.complex128)
    c = np.array([100.0005 + 0j, 0.00130 + 0j, 0.001 + 0j, 0.001 + 0j], dtype=np.complex64)   # second: CPU off by 3e-4
    S = np.array([500.0, 500.0, 500.0, 500.0])
    g = np.array([100.0008 + 0j,      # A: within 1e-5 relative of the CPU value
                  0.00090 + 0j,       # B: the CPU misses its own gate, the GPU is closer to the exact value
                  0.00105 + 0j,       # C: 5e-5 from exact, under 1e-6 + 2 eps32 * 500 = 1.2e-4
                  0.00150 + 0j],      # rejected: 5e-4 from exact and from the CPU
                 dtype=np.complex64)
    rep = U.parity_counts(g, c, e, S)
    assert rep["rejected"] == 1 and rep["first_rejected"] == 6
    assert rep["by_rule_B"] == 1 / 8 and rep["by_rule_C"] == 1 / 8
    with pytest.raises(AssertionError):
        U.assert_parity(g, c, e, S, "demo")
    U.assert_parity(g[:3], c[:3], e[:3], S[:3], "demo")
