"""Randomly drawn products (fixed seeds) through the C-ABI against the CPU oracle: any mix of parts, channel counts,
caps, batch broadcasting, Diag or not, accumulate or overwrite.  Whatever kernel family the library picks for a draw,
the result has to agree with the oracle; the draws are spread so that every family gets its share."""
import numpy as np
import pytest

from oracle import cg_oracle as ora
from tests import gpu_util as U

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def cabi():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from gelib_amd import cabi as c
    c.lib()
    for name in ("diag6", "onepair", "unrolled_fwd", "unrolled_bwd", "staged_fwd", "staged_bwd"):
        c.set_option(name, 1)
    c.set_option("force_generic", 0)
    return c


def c128(L):
    return [a.astype(np.complex128) for a in L]


def draw(rng):
    diag = bool(rng.integers(0, 2))
    lmax = int(rng.choice([2, 4, 6, 8, 10]))
    nparts = int(rng.integers(1, 4))
    lx = sorted(rng.choice(lmax + 1, size=min(nparts, lmax + 1), replace=False).tolist())
    ly = sorted(rng.choice(lmax + 1, size=min(int(rng.integers(1, 4)), lmax + 1), replace=False).tolist())
    if diag:
        n = int(rng.choice([1, 3, 8, 16, 24, 33, 64, 70]))
        tx, ty = {l: n for l in lx}, {l: n for l in ly}
    else:
        same = bool(rng.integers(0, 2))
        pick = lambda: int(rng.choice([1, 2, 3, 4, 5, 8, 12, 16]))
        nx, ny = pick(), pick()
        tx = {l: (nx if same else pick()) for l in lx}
        ty = {l: (ny if same else pick()) for l in ly}
    top = max(lx) + max(ly)
    maxl = int(rng.choice([-1, -1, top // 2, max(0, top - 1)]))
    lo = min(abs(a - b) for a in lx for b in ly)
    if 0 <= maxl < lo:
        maxl = lo
    B = int(rng.choice([1, 2, 5, 9, 33, 70]))
    bx = 1 if rng.integers(0, 5) == 0 else B      # sometimes x is shared by the whole batch
    return B, bx, tx, ty, maxl, diag


@pytest.mark.parametrize("seed", range(160))
def test_random_product(cabi, seed):
    rng = np.random.default_rng(7000 + seed)
    B, bx, tx, ty, maxl, diag = draw(rng)
    xs = [U.seeded(seed * 10 + l, bx, 2 * l + 1, n) for l, n in sorted(tx.items())]
    ys = [U.seeded(seed * 10 + 50 + l, B, 2 * l + 1, n) for l, n in sorted(ty.items())]
    bxs = [np.broadcast_to(a, (B,) + a.shape[1:]) for a in xs]
    r32 = ora.vec_fwd(bxs, ys, maxl, diag)
    r64 = ora.vec_fwd(c128(bxs), c128(ys), maxl, diag)
    tag = "seed %d: B %d bx %d %s x %s maxl %d diag %d" % (seed, B, bx, tx, ty, maxl, diag)
    dxs, dys = [U.dev(a) for a in xs], [U.dev(a) for a in ys]
    start = [U.seeded(seed + 300 + i, *p.shape) for i, p in enumerate(r32)]
    accumulate = bool(rng.integers(0, 2))
    drs = [U.dev(a) for a in start]
    cabi.so3vec_fwd(drs, dxs, dys, accumulate=accumulate, diag=diag)
    torch.cuda.synchronize()
    for a, s, b, c in zip(drs, start, r32, r64):
        got = U.host(a) - (s if accumulate else 0)
        U.assert_parity(got, b, c, "fwd " + tag + " path %d" % cabi.last_path(), slack=4.0)
    # both gradients; a broadcast x gets none (its gradient is a sum over the batch, a different call)
    gs = [U.seeded(seed + 100 + i, *p.shape) for i, p in enumerate(r32)]
    xg32, yg32 = ora.vec_bwd(gs, bxs, ys, diag)
    xg64, yg64 = ora.vec_bwd(c128(gs), c128(bxs), c128(ys), diag)
    dgs = [U.dev(a) for a in gs]
    dyg = [torch.full(a.shape, 2.0 + 1j, dtype=torch.complex64, device="cuda") for a in ys]
    dxg = None if bx != B else [torch.full(a.shape, 2.0 + 1j, dtype=torch.complex64, device="cuda") for a in xs]
    cabi.so3vec_bwd(dxg, dyg, dgs, dxs, dys, accumulate=False, diag=diag)
    torch.cuda.synchronize()
    path = cabi.last_path()
    for a, b, c in zip(dyg, yg32, yg64):
        U.assert_parity(U.host(a), b, c, "yg " + tag + " path %d" % path, slack=4.0)
    if dxg is not None:
        for a, b, c in zip(dxg, xg32, xg64):
            U.assert_parity(U.host(a), b, c, "xg " + tag + " path %d" % path, slack=4.0)
