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
