"""GPU parity of the fused CGproduct -> weight matrices entry point (gelib_hip_so3vec_cg_linear_fwd) against the CPU
oracle's product followed by numpy matmuls, and of the Python function built on it (values and gradients).

The check per real component is the one of the product tests: inside the 1e-6 + 1e-5 |c| gate of the float32 CPU result
(oracle product, complex64 matmul), or at least as close to the float64 result as that one where it sits outside the gate
itself, or within 2 eps32 times the sum of the moduli of the terms.  The terms of a component here are those of the
product's element, sum |C| |x| |y|, times |Re W| + |Im W| of the matrix element they meet."""
import numpy as np
import pytest

from tests import gpu_util as U

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def cabi():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from gelib_amd import cabi as c
    c.lib()
    return c


def weights(seed, taus, nouts):
    return [U.seeded(seed + l, taus[l], nouts[l], scale=1.0 / np.sqrt(max(taus[l], 1))) for l in range(len(taus))]


def oracle_linear(O, ws):
    """float32, float64 and term-sum results of (product) @ W per part."""
    r32 = [np.matmul(p, w) for p, w in zip(O.r32, ws)]
    r64 = [np.matmul(p, w.astype(np.complex128)) for p, w in zip(O.r64, ws)]
    S = [np.matmul(s, (np.abs(w.real) + np.abs(w.imag)).astype(np.float64)) for s, w in zip(O.Sr, ws)]
    return r32, r64, S


CASES = [
    # (B, tau_x, tau_y, n_out per l)
    (33, {l: 16 for l in range(5)}, {l: 16 for l in range(5)}, [16] * 5),   # headline type, a partial last block
    (64, {l: 16 for l in range(5)}, {l: 16 for l in range(5)}, [16, 8, 4, 2, 1]),
    (5, {l: 3 for l in range(5)}, {l: 5 for l in range(5)}, [7, 16, 3, 1, 9]),
    (40, {2: 4}, {2: 6}, [5] * 5),                                           # one pair reaches every l
    (7, {0: 2, 2: 3, 4: 1}, {1: 4, 2: 2, 3: 5}, [4, 6, 8, 10, 12]),
    (1, {l: 16 for l in range(5)}, {l: 16 for l in range(5)}, [16] * 5),
]


@pytest.mark.parametrize("case", CASES, ids=[str(i) for i in range(len(CASES))])
def test_fused_forward_matches_product_then_matmul(cabi, case):
    B, tx, ty, nouts = case
    seed = 4100 + B
    xs = [U.seeded(seed + l, B, 2 * l + 1, n) for l, n in sorted(tx.items())]
    ys = [U.seeded(seed + 50 + l, B, 2 * l + 1, n) for l, n in sorted(ty.items())]
    O = U.VecOracle(xs, ys, 4, False)
    taus = [p.shape[2] for p in O.r32]
    assert len(taus) == 5
    ws = weights(seed + 200, taus, nouts)
    r32, r64, S = oracle_linear(O, ws)
    dxs, dys, dws = [U.dev(a) for a in xs], [U.dev(a) for a in ys], [U.dev(a) for a in ws]
    outs = [torch.full((B, 2 * l + 1, nouts[l]), 7.0 + 1j, dtype=torch.complex64, device="cuda") for l in range(5)]
    assert cabi.so3vec_cg_linear_fwd(outs, dxs, dys, dws, accumulate=False)
    assert cabi.last_path() == 6
    torch.cuda.synchronize()
    tag = "linear B%d %s x %s -> %s" % (B, tx, ty, nouts)
    for l in range(5):
        U.assert_parity(U.host(outs[l]), r32[l], r64[l], S[l], tag + " l=%d" % l)
    # accumulate mode adds onto what is there; parts handed over in another order
    start = [U.seeded(seed + 300 + l, B, 2 * l + 1, nouts[l]) for l in range(5)]
    outs2 = [U.dev(a) for a in start]
    order = [3, 0, 4, 1, 2]
    assert cabi.so3vec_cg_linear_fwd([outs2[k] for k in order], dxs[::-1], dys, [dws[k] for k in order], accumulate=True)
    torch.cuda.synchronize()
    for l in range(5):
        U.assert_parity(U.host(outs2[l]), (r32[l] + start[l]).astype(np.complex64), r64[l] + start[l],
                        S[l] + np.abs(start[l]), tag + " onto l=%d" % l)
    # two runs give the same bits
    outs3 = [torch.empty_like(t) for t in outs]
    assert cabi.so3vec_cg_linear_fwd(outs3, dxs, dys, dws, accumulate=False)
    torch.cuda.synchronize()
    assert all(torch.equal(a.view(torch.float32), b.view(torch.float32)) for a, b in zip(outs, outs3))


def test_grid_dimensions_collapse_into_cells(cabi):
    """Parts with grid dimensions (batch, grid0, grid1, 2l+1, n), contiguous: 3 x 4 x 5 = 60 cells."""
    lead, n, n_out = (3, 4, 5), 4, 6
    B = 60
    xs = [U.seeded(700 + l, B, 2 * l + 1, n) for l in range(5)]
    ys = [U.seeded(750 + l, B, 2 * l + 1, n) for l in range(5)]
    O = U.VecOracle(xs, ys, 4, False)
    taus = [p.shape[2] for p in O.r32]
    ws = weights(800, taus, [n_out] * 5)
    r32, r64, S = oracle_linear(O, ws)
    dxs = [U.dev(a).reshape(*lead, 2 * l + 1, n) for l, a in enumerate(xs)]
    dys = [U.dev(a).reshape(*lead, 2 * l + 1, n) for l, a in enumerate(ys)]
    dws = [U.dev(a) for a in ws]
    outs = [torch.full((*lead, 2 * l + 1, n_out), 7.0 + 1j, dtype=torch.complex64, device="cuda") for l in range(5)]
    assert cabi.so3vec_cg_linear_fwd(outs, dxs, dys, dws, accumulate=False)
    torch.cuda.synchronize()
    for l in range(5):
        U.assert_parity(U.host(outs[l]).reshape(B, 2 * l + 1, n_out), r32[l], r64[l], S[l], "grid l=%d" % l)
    # an operand that broadcasts over the grid is not a case of the fused kernel
    bx = [t[:, :1, :1].expand(*lead, -1, -1) for t in dxs]
    assert cabi.so3vec_cg_linear_fwd(outs, bx, dys, dws, accumulate=False) is False


def test_shapes_the_fused_kernel_does_not_take(cabi):
    B = 4
    xs = [U.dev(U.seeded(1 + l, B, 2 * l + 1, 4)) for l in range(3)]
    ys = [U.dev(U.seeded(9 + l, B, 2 * l + 1, 4)) for l in range(3)]
    # a product without l = 4
    outs = [torch.zeros((B, 2 * l + 1, 4), dtype=torch.complex64, device="cuda") for l in range(4)]
    ws = [torch.zeros((16 * 9, 4), dtype=torch.complex64, device="cuda") for l in range(4)]
    assert cabi.so3vec_cg_linear_fwd(outs, xs, ys, ws) is False
    # more than 16 output channels
    outs = [torch.zeros((B, 2 * l + 1, 17), dtype=torch.complex64, device="cuda") for l in range(5)]
    ws = [torch.zeros((16 * 9, 17), dtype=torch.complex64, device="cuda") for l in range(5)]
    assert cabi.so3vec_cg_linear_fwd(outs, xs, ys, ws) is False
    torch.cuda.synchronize()
    assert all(float(o.abs().max()) == 0.0 for o in outs)


def test_workspace_rules(cabi):
    import ctypes
    B = 3
    xs = [U.dev(U.seeded(1 + l, B, 2 * l + 1, 2)) for l in range(5)]
    ys = [U.dev(U.seeded(9 + l, B, 2 * l + 1, 2)) for l in range(5)]
    taus = cabi.so3type_product({l: 2 for l in range(5)}, {l: 2 for l in range(5)}, 4)
    outs = [torch.zeros((B, 2 * l + 1, 2), dtype=torch.complex64, device="cuda") for l in range(5)]
    ws = [torch.zeros((taus[l], 2), dtype=torch.complex64, device="cuda") for l in range(5)]
    L = cabi.lib()
    ra, xa, ya = cabi._arr(outs), cabi._arr(xs), cabi._arr(ys)
    need = int(L.gelib_hip_so3vec_cg_linear_workspace_bytes(5, ra, 5, xa, 5, ya))
    # the packed matrices (16 channels of padding per part) and x transposed, rounded up to a group of 32 cells
    assert need == sum((taus[l] + 16) * 256 for l in range(5)) + 32 * sum((2 * l + 1) * 2 for l in range(5)) * 8
    wp = (ctypes.c_void_p * 5)(*[w.data_ptr() for w in ws])
    buf = torch.empty(need, dtype=torch.uint8, device="cuda")
    st = cabi._stream(outs[0])
    call = lambda p, n: L.gelib_hip_so3vec_cg_linear_fwd(5, ra, 5, xa, 5, ya, wp, 0, ctypes.c_void_p(p), n, st)
    assert call(buf.data_ptr(), need) == 0
    assert call(buf.data_ptr(), need - 256) == 13
    assert call(0, need) == 13
    assert call(buf.data_ptr() + 4, need) == 13
    torch.cuda.synchronize()


def test_python_function_values_and_gradients(cabi):
    import gelib_amd as gelib
    B = 6
    tau = {l: 4 for l in range(5)}
    torch.manual_seed(11)
    x = gelib.SO3vec.randn(B, tau, device="cuda")
    y = gelib.SO3vec.randn(B, tau, device="cuda")
    taus = gelib.SO3type(cabi.so3type_product(tau, tau, 4))
    W = gelib.SO3weights.randn(taus, gelib.SO3type({l: 8 for l in range(5)}), device="cuda")
    for v in (x, y, W):
        v.requires_grad_()
    fused = gelib.CGproduct_linear(x, y, W, maxl=4)
    assert cabi.last_path() == 6
    plain = gelib.CGproduct(x, y, maxl=4) * W
    coef = [torch.randn_like(p) for p in plain.parts.values()]
    leaves = list(x.parts.values()) + list(y.parts.values()) + list(W.parts)
    loss = lambda v: sum((p * c).real.sum() for p, c in zip(v.parts.values(), coef))
    g_fused = torch.autograd.grad(loss(fused), leaves)
    g_plain = torch.autograd.grad(loss(plain), leaves)
    for l in range(5):
        a, b = fused.parts[l].detach(), plain.parts[l].detach()
        assert float((a - b).abs().max()) <= 2e-5 * float(b.abs().max()), l
    for a, b in zip(g_fused, g_plain):   # the backward pass of the fused function runs the unfused kernels
        assert torch.equal(a, b)
    # a case outside the fused kernel goes through the two steps and gives the same as writing them out
    W17 = gelib.SO3weights.randn(taus, gelib.SO3type({l: 17 for l in range(5)}), device="cuda")
    two = gelib.CGproduct_linear(x, y, W17, maxl=4)
    ref = gelib.CGproduct(x, y, maxl=4) * W17
    assert all(torch.equal(two.parts[l], ref.parts[l]) for l in range(5))


BWD_CASES = [
    # (B, tau_x, tau_y, maxl, n_out per product part)
    (33, {l: 16 for l in range(5)}, {l: 16 for l in range(5)}, 4, [16] * 5),     # headline type
    (20, {l: 4 for l in range(5)}, {l: 4 for l in range(5)}, 4, [8, 2, 4, 6, 16]),
    (9, {0: 2, 2: 4}, {1: 4, 3: 2}, -1, [4] * 5),                                 # not a case of the fused forward kernel
    (6, {l: 8 for l in range(3)}, {l: 8 for l in range(3)}, 2, [32, 32, 32]),
]


@pytest.mark.parametrize("case", BWD_CASES, ids=[str(i) for i in range(len(BWD_CASES))])
def test_linear_backward_in_bounded_memory(cabi, case):
    """gelib_hip_so3vec_cg_linear_bwd against float64: gP = g W^H and the matrix gradient sum P^H g from numpy complex128
    on the oracle's float64 product, the gradients of x and y from the oracle's float64 backward loops on gP.  Bound per
    real component: 1e-6 + 8 eps32 S with S the sum of the moduli of the element's terms (the oracle's loops on moduli,
    through |g| |W|^T for the operands' gradients and through the product's own term sums for the matrices'): the
    sums run in float32 in another order than any CPU evaluation, and a dropped or misplaced term is 1e4 times larger."""
    from oracle import cg_oracle as ora
    B, tx, ty, maxl, nouts = case
    seed = 5200 + B
    xs = [U.seeded(seed + l, B, 2 * l + 1, n) for l, n in sorted(tx.items())]
    ys = [U.seeded(seed + 50 + l, B, 2 * l + 1, n) for l, n in sorted(ty.items())]
    O = U.VecOracle(xs, ys, maxl, False)
    ls = [(p.shape[1] - 1) // 2 for p in O.r32]
    taus = [p.shape[2] for p in O.r32]
    assert len(taus) == len(nouts)
    ws = weights(seed + 200, taus, nouts)
    gs = [U.seeded(seed + 300 + k, B, 2 * l + 1, nouts[k]) for k, l in enumerate(ls)]
    w64 = [w.astype(np.complex128) for w in ws]
    g64 = [g.astype(np.complex128) for g in gs]
    gP64 = [np.matmul(g, w.conj().T) for g, w in zip(g64, w64)]
    xg64, yg64 = ora.vec_bwd(gP64, U.c128(xs), U.c128(ys))
    wg64 = [np.einsum("bmc,bmo->co", p.conj(), g) for p, g in zip(O.r64, g64)]
    gPabs = [np.matmul(np.abs(g), np.abs(w).T).astype(np.complex128) for g, w in zip(g64, w64)]
    Sx, Sy = ora.vec_bwd_term_sums(gPabs, xs, ys)
    Sw = [np.einsum("bmc,bmo->co", s, np.abs(g)) for s, g in zip(O.Sr, g64)]

    def close(got, exact, S, what):
        err = np.abs(U.components(got).astype(np.float64) - U.components(np.asarray(exact, dtype=np.complex128)))
        bound = 1e-6 + 8 * U.EPS32 * np.repeat(np.asarray(S, dtype=np.float64).reshape(-1), 2).reshape(err.shape)
        assert np.all(err <= bound), "%s: worst error / bound %.3f" % (what, float(np.max(err / bound)))

    dxs, dys, dws, dgs = ([U.dev(a) for a in L] for L in (xs, ys, ws, gs))
    tag = "linear bwd B%d %s x %s maxl %d -> %s" % (B, tx, ty, maxl, nouts)

    def run(ws_bytes, acc=False, start=None, want=(True, True, True)):
        mk = lambda L, k: ([U.dev(a) for a in start[k]] if start else
                           [torch.full(a.shape, 3.0 - 2j, dtype=torch.complex64, device="cuda") for a in L])
        xg, yg, wg = mk(xs, 0), mk(ys, 1), mk(ws, 2)
        ok = cabi.so3vec_cg_linear_bwd(xg if want[0] else None, yg if want[1] else None, wg if want[2] else None, dgs, dxs,
                                       dys, dws, accumulate=acc, workspace_bytes=ws_bytes)
        assert ok
        torch.cuda.synchronize()
        return [U.host(a) for a in xg], [U.host(a) for a in yg], [U.host(a) for a in wg]

    xg, yg, wg = run(1 << 30)
    for k in range(len(xs)):
        close(xg[k], xg64[k], Sx[k], tag + " xg[%d]" % k)
    for k in range(len(ys)):
        close(yg[k], yg64[k], Sy[k], tag + " yg[%d]" % k)
    for k in range(len(ws)):
        close(wg[k], wg64[k], Sw[k], tag + " wg[%d]" % k)
    # a workspace that holds a few batch entries only: several chunks, the matrix gradient summed over them
    L = cabi.lib()
    one = int(L.gelib_hip_so3vec_cg_linear_bwd_workspace_bytes(len(dgs), cabi._arr(dgs), len(dxs), cabi._arr(dxs), len(dys),
                                                               cabi._arr(dys), 1))
    whole = int(L.gelib_hip_so3vec_cg_linear_bwd_workspace_bytes(len(dgs), cabi._arr(dgs), len(dxs), cabi._arr(dxs),
                                                                 len(dys), cabi._arr(dys), 0))
    assert 0 < one < whole
    xg2, yg2, wg2 = run(one + (whole - one) // 7)
    for k in range(len(xs)):
        close(xg2[k], xg64[k], Sx[k], tag + " chunked xg[%d]" % k)
    for k in range(len(ys)):
        close(yg2[k], yg64[k], Sy[k], tag + " chunked yg[%d]" % k)
    for k in range(len(ws)):
        close(wg2[k], wg64[k], Sw[k], tag + " chunked wg[%d]" % k)
    # accumulate mode, chunked: onto given starting values
    start = ([U.seeded(seed + 400 + k, *a.shape) for k, a in enumerate(xs)],
             [U.seeded(seed + 420 + k, *a.shape) for k, a in enumerate(ys)],
             [U.seeded(seed + 440 + k, *a.shape) for k, a in enumerate(ws)])
    xg3, yg3, wg3 = run(one + (whole - one) // 3, acc=True, start=start)
    for k in range(len(xs)):
        close(xg3[k], xg64[k] + start[0][k], Sx[k] + np.abs(start[0][k]), tag + " onto xg[%d]" % k)
    for k in range(len(ys)):
        close(yg3[k], yg64[k] + start[1][k], Sy[k] + np.abs(start[1][k]), tag + " onto yg[%d]" % k)
    for k in range(len(ws)):
        close(wg3[k], wg64[k] + start[2][k], Sw[k] + np.abs(start[2][k]), tag + " onto wg[%d]" % k)
    # one kind of gradient per call: what is not asked for is not touched
    xg4, yg4, wg4 = run(1 << 30, want=(False, False, True))
    assert all(np.all(a == np.complex64(3.0 - 2j)) for a in xg4 + yg4)
    assert all(np.array_equal(a, b) for a, b in zip(wg4, wg))
    xg5, yg5, wg5 = run(1 << 30, want=(True, True, False))
    assert all(np.all(a == np.complex64(3.0 - 2j)) for a in wg5)
    assert all(np.array_equal(a, b) for a, b in zip(xg5 + yg5, xg + yg))


def test_linear_backward_declines_and_workspace_rules(cabi):
    import ctypes
    B = 4
    xs = [U.dev(U.seeded(1 + l, B, 2 * l + 1, 3)) for l in range(2)]     # 3 x 3 = 9 product channels per pair: odd counts
    ys = [U.dev(U.seeded(9 + l, B, 2 * l + 1, 3)) for l in range(2)]
    taus = cabi.so3type_product({0: 3, 1: 3}, {0: 3, 1: 3}, -1)
    gs = [torch.zeros((B, 2 * l + 1, 4), dtype=torch.complex64, device="cuda") for l in sorted(taus)]
    ws = [torch.zeros((taus[l], 4), dtype=torch.complex64, device="cuda") for l in sorted(taus)]
    xg, yg = [torch.zeros_like(t) for t in xs], [torch.zeros_like(t) for t in ys]
    assert cabi.so3vec_cg_linear_bwd(xg, yg, None, gs, xs, ys, ws) is False      # tau_0 = 9 + 9 = 18 is even, tau_2 = 9 is odd
    xs = [U.dev(U.seeded(1 + l, B, 2 * l + 1, 2)) for l in range(2)]
    ys = [U.dev(U.seeded(9 + l, B, 2 * l + 1, 2)) for l in range(2)]
    taus = cabi.so3type_product({0: 2, 1: 2}, {0: 2, 1: 2}, -1)
    ws = [torch.zeros((taus[l], 4), dtype=torch.complex64, device="cuda") for l in sorted(taus)]
    xg, yg = [torch.zeros_like(t) for t in xs], [torch.zeros_like(t) for t in ys]
    L = cabi.lib()
    ga, xa, ya = cabi._arr(gs), cabi._arr(xs), cabi._arr(ys)
    one = int(L.gelib_hip_so3vec_cg_linear_bwd_workspace_bytes(3, ga, 2, xa, 2, ya, 1))
    assert one > 0
    buf = torch.empty(one + 512, dtype=torch.uint8, device="cuda")
    base = (buf.data_ptr() + 255) & ~255
    wp = (ctypes.c_void_p * 3)(*[w.data_ptr() for w in ws])
    call = lambda p, n: L.gelib_hip_so3vec_cg_linear_bwd(cabi._arr(xg), cabi._arr(yg), None, 3, ga, 2, xa, 2, ya, wp, 0,
                                                         ctypes.c_void_p(p), n, cabi._stream(gs[0]))
    assert call(base, one) == 0
    assert call(base, one - 256) == 13       # not even one batch entry fits
    assert call(base + 16, one) == 13        # 256-byte alignment
    assert call(0, one) == 13
    torch.cuda.synchronize()
