"""Gradients whose destination broadcasts (an operand shared by the batch or by the grid, core/Gpart.hpp:168-185; the
reference's CI exercises it in python/tests/ci_tests/test_SO3part.py:31-52,103-107): the library writes one gradient per
cell into its own temporary and sums those in a fixed order.  Checked against the oracle's serial sum over the broadcast
dimension (the reference's loop order) under the parity rules, whose term sums then run over the summed cells too."""
import numpy as np
import pytest

from oracle import cg_oracle as ora
from tests import gpu_util as U

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

GENERIC, UNROLLED, STAGED, DIAG6 = 1, 2, 3, 4


@pytest.fixture(scope="module")
def cabi():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from gelib_amd import cabi as c
    c.lib()
    yield c
    c.set_option("bcast_scratch_kb", 0)
    c.set_option("bcast_reduce", 1)
    c.set_option("force_generic", 0)


def make(B, tx, ty, shared, seed):
    bx, by = (1, B) if shared == "x" else (B, 1) if shared == "y" else (1, 1)
    xs = [U.seeded(seed + l, bx, 2 * l + 1, n) for l, n in sorted(tx.items())]
    ys = [U.seeded(seed + 50 + l, by, 2 * l + 1, n) for l, n in sorted(ty.items())]
    return xs, ys


CASES = [
    # (B, tau_x, tau_y, maxl, diag, family expected for the per-cell pass)
    (300, {0: 4, 1: 4, 2: 4}, {0: 4, 1: 4, 2: 4}, 2, False, UNROLLED),
    (257, {l: 16 for l in range(5)}, {l: 16 for l in range(5)}, 4, False, UNROLLED),   # headline type
    (90, {0: 3, 1: 2, 2: 5}, {1: 2, 2: 3}, -1, False, UNROLLED),
    (130, {l: 8 for l in range(4)}, {l: 8 for l in range(4)}, 3, True, DIAG6),
    (40, {l: 64 for l in range(3)}, {l: 64 for l in range(3)}, -1, True, DIAG6),
    (24, {8: 4}, {7: 2, 9: 2}, 10, False, None),
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("shared", ["x", "y"])
def test_vec_shared_operand(cabi, case, shared):
    B, tx, ty, maxl, diag, family = case
    cabi.set_option("force_generic", 0)
    cabi.set_option("bcast_scratch_kb", 0)
    xs, ys = make(B, tx, ty, shared, 1000)
    gtmpl = ora.vec_fwd(xs, ys, maxl, diag)
    gs = [U.seeded(2000 + i, *p.shape) for i, p in enumerate(gtmpl)]
    O = U.VecOracle(xs, ys, maxl, diag, gs=gs)
    dxs, dys, dgs = [U.dev(a) for a in xs], [U.dev(a) for a in ys], [U.dev(a) for a in gs]

    def run(acc, start=None):
        dxg = [torch.full(a.shape, 3.0 - 2j, dtype=torch.complex64, device="cuda") if start is None else U.dev(s)
               for a, s in zip(xs, start[0] if start else xs)]
        dyg = [torch.full(a.shape, 3.0 - 2j, dtype=torch.complex64, device="cuda") if start is None else U.dev(s)
               for a, s in zip(ys, start[1] if start else ys)]
        cabi.so3vec_bwd(dxg, dyg, dgs, dxs, dys, accumulate=acc, diag=diag)
        path = cabi.last_path()
        torch.cuda.synchronize()
        return [U.host(a) for a in dxg], [U.host(a) for a in dyg], path

    xg, yg, path = run(False)
    tag = "B%d %s x %s maxl %d diag %d shared %s" % (B, tx, ty, maxl, diag, shared)
    assert xg[0].shape[0] == (1 if shared == "x" else B) and yg[0].shape[0] == (1 if shared == "y" else B)
    O.check_bwd(xg, yg, tag)
    if family is not None:
        assert path == family, "per-cell pass ran on family %d" % path
    # the same bits on a second run, and with the batch cut into chunks by a small temporary
    xg2, yg2, _ = run(False)
    assert all(np.array_equal(a, b) for a, b in zip(xg + yg, xg2 + yg2))
    cabi.set_option("bcast_scratch_kb", 16)
    xg3, yg3, _ = run(False)
    O.check_bwd(xg3, yg3, tag + " chunked")
    # accumulate mode: onto given starting values (with chunks: every chunk adds onto the one before)
    sx = [U.seeded(3000 + i, *a.shape) for i, a in enumerate(xs)]
    sy = [U.seeded(3100 + i, *a.shape) for i, a in enumerate(ys)]
    xg4, yg4, _ = run(True, (sx, sy))
    O.check_bwd_onto(xg4, yg4, sx, sy, tag + " accumulate")
    cabi.set_option("bcast_scratch_kb", 0)
    # the in-thread serial sum of the shape-agnostic kernels gives the same to rounding
    cabi.set_option("bcast_reduce", 0)
    xg5, yg5, path5 = run(False)
    cabi.set_option("bcast_reduce", 1)
    assert path5 == GENERIC
    O.check_bwd(xg5, yg5, tag + " serial")


def test_one_gradient_only_and_both_shared(cabi):
    cabi.set_option("force_generic", 0)
    B, tau = 50, {0: 4, 1: 4, 2: 4}
    xs, ys = make(B, tau, tau, "x", 50)
    gs = [U.seeded(60 + i, *p.shape) for i, p in enumerate(ora.vec_fwd(xs, ys, 2))]
    O = U.VecOracle(xs, ys, 2, False, gs=gs)
    dxs, dys, dgs = [U.dev(a) for a in xs], [U.dev(a) for a in ys], [U.dev(a) for a in gs]
    dxg = [torch.empty_like(a) for a in dxs]
    cabi.so3vec_bwd(dxg, None, dgs, dxs, dys, accumulate=False)
    torch.cuda.synchronize()
    O.check_bwd([U.host(a) for a in dxg], None, "back0 only")
    dyg = [torch.empty_like(a) for a in dys]
    cabi.so3vec_bwd(None, dyg, dgs, dxs, dys, accumulate=False)
    torch.cuda.synchronize()
    O.check_bwd(None, [U.host(a) for a in dyg], "back1 only")
    # both operands shared by the batch: g alone carries the batch
    xs1, ys1 = make(B, tau, tau, "both", 70)
    O1 = U.VecOracle(xs1, ys1, 2, False, gs=gs)
    dx1, dy1 = [U.dev(a) for a in xs1], [U.dev(a) for a in ys1]
    dxg1, dyg1 = [torch.empty_like(a) for a in dx1], [torch.empty_like(a) for a in dy1]
    cabi.so3vec_bwd(dxg1, dyg1, dgs, dx1, dy1, accumulate=False)
    torch.cuda.synchronize()
    O1.check_bwd([U.host(a) for a in dxg1], [U.host(a) for a in dyg1], "both shared")


@pytest.mark.parametrize("diag", [False, True])
@pytest.mark.parametrize("xdims", [(5, 1, 1), (1, 3, 1), (1, 1, 1), (5, 1, 4)])
def test_part_level_grid_and_batch(cabi, diag, xdims):
    """Part-level back0 with the destination broadcast over any of (batch, grid0, grid1).  The oracle knows batches
    only: for every cell of the destination the summed cells are handed to it as a batch, in the reference's order
    (batch slowest)."""
    cabi.set_option("force_generic", 0)
    E = (5, 3, 4)
    l1, l2, l, n = 2, 1, 2, 4
    x = U.seeded(1, *xdims, 2 * l1 + 1, n)
    y = U.seeded(2, *E, 2 * l2 + 1, n)
    g = U.seeded(3, *E, 2 * l + 1, n if diag else n * n)
    op = ora.DIAG_BACK0 if diag else ora.CG_BACK0
    want32 = np.zeros_like(x)
    want64 = np.zeros(x.shape, dtype=np.complex128)
    S = np.zeros(x.shape)
    for c in np.ndindex(*xdims):
        sel = tuple(slice(None) if xdims[k] == 1 else slice(c[k], c[k] + 1) for k in range(3))
        gc = np.ascontiguousarray(g[sel]).reshape(-1, *g.shape[3:])
        yc = np.ascontiguousarray(y[sel]).reshape(-1, *y.shape[3:])
        xc = np.ascontiguousarray(x[c])[None]
        o32 = np.zeros_like(xc)
        ora.part_op(op, gc, o32, yc)
        o64 = np.zeros(xc.shape, dtype=np.complex128)
        ora.part_op(op, gc.astype(np.complex128), o64, yc.astype(np.complex128))
        want32[c], want64[c] = o32[0], o64[0]
        S[c] = ora.part_term_sums(op, gc, xc, yc)[0]
    dxg = torch.full(x.shape, 5.0 + 1j, dtype=torch.complex64, device="cuda")
    fn = cabi.so3part_diagcg_back0 if diag else cabi.so3part_cg_back0
    fn(dxg, U.dev(g), U.dev(y), accumulate=False)
    assert cabi.last_path() != GENERIC
    torch.cuda.synchronize()
    U.assert_parity(U.host(dxg), want32, want64, S, "part back0 xdims %s diag %d" % (xdims, diag))
    # back1 with the roles swapped: y shared, x per cell
    yb = U.seeded(4, *xdims, 2 * l2 + 1, n)
    xb = U.seeded(5, *E, 2 * l1 + 1, n)
    op1 = ora.DIAG_BACK1 if diag else ora.CG_BACK1
    w32 = np.zeros_like(yb)
    w64 = np.zeros(yb.shape, dtype=np.complex128)
    S1 = np.zeros(yb.shape)
    start = U.seeded(6, *yb.shape)
    for c in np.ndindex(*xdims):
        sel = tuple(slice(None) if xdims[k] == 1 else slice(c[k], c[k] + 1) for k in range(3))
        gc = np.ascontiguousarray(g[sel]).reshape(-1, *g.shape[3:])
        xc = np.ascontiguousarray(xb[sel]).reshape(-1, *xb.shape[3:])
        yc = np.ascontiguousarray(yb[c])[None]
        o32 = np.ascontiguousarray(start[c])[None].copy()      # the reference adds its terms onto what is there
        ora.part_op(op1, gc, xc, o32)
        o64 = np.ascontiguousarray(start[c])[None].astype(np.complex128)
        ora.part_op(op1, gc.astype(np.complex128), xc.astype(np.complex128), o64)
        w32[c], w64[c] = o32[0], o64[0]
        S1[c] = ora.part_term_sums(op1, gc, xc, yc)[0]
    dyg = U.dev(start)
    fn1 = cabi.so3part_diagcg_back1 if diag else cabi.so3part_cg_back1
    fn1(dyg, U.dev(g), U.dev(xb), accumulate=True)
    torch.cuda.synchronize()
    U.assert_parity(U.host(dyg), w32, w64, S1 + np.abs(start),
                    "part back1 onto a start, ydims %s diag %d" % (xdims, diag))
