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
    O = U.VecOracle(xs, ys, maxl, diag, gseed=seed + 100)    # an x of batch 1 is shared by the batch, in the oracle too
    r32, gs = O.r32, O.gs
    tag = "seed %d: B %d bx %d %s x %s maxl %d diag %d" % (seed, B, bx, tx, ty, maxl, diag)
    dxs, dys = [U.dev(a) for a in xs], [U.dev(a) for a in ys]
    start = [U.seeded(seed + 300 + i, *p.shape) for i, p in enumerate(r32)]
    accumulate = bool(rng.integers(0, 2))
    drs = [U.dev(a) for a in start]
    cabi.so3vec_fwd(drs, dxs, dys, accumulate=accumulate, diag=diag)
    torch.cuda.synchronize()
    what = tag + " path %d" % cabi.last_path()
    if accumulate:
        O.check_fwd_onto([U.host(a) for a in drs], start, what)
    else:
        O.check_fwd([U.host(a) for a in drs], what)
    # both gradients; that of an x shared by the batch is the sum over the batch (formed inside the library)
    dgs = [U.dev(a) for a in gs]
    dyg = [torch.full(a.shape, 2.0 + 1j, dtype=torch.complex64, device="cuda") for a in ys]
    dxg = [torch.full(a.shape, 2.0 + 1j, dtype=torch.complex64, device="cuda") for a in xs]
    cabi.so3vec_bwd(dxg, dyg, dgs, dxs, dys, accumulate=False, diag=diag)
    torch.cuda.synchronize()
    path = cabi.last_path()
    O.check_bwd(None if dxg is None else [U.host(a) for a in dxg], [U.host(a) for a in dyg], tag + " path %d" % path)
    # no kernel on the default dispatch adds with atomics: a second run gives the same bits, forward and backward
    drs2 = [U.dev(a) for a in start]
    cabi.so3vec_fwd(drs2, dxs, dys, accumulate=accumulate, diag=diag)
    dyg2 = [torch.full_like(a, 2.0 + 1j) for a in dyg]
    dxg2 = None if dxg is None else [torch.full_like(a, 2.0 + 1j) for a in dxg]
    cabi.so3vec_bwd(dxg2, dyg2, dgs, dxs, dys, accumulate=False, diag=diag)
    torch.cuda.synchronize()
    for a, b in zip(drs + dyg + (dxg or []), drs2 + dyg2 + (dxg2 or [])):
        assert torch.equal(torch.view_as_real(a), torch.view_as_real(b)), tag + " path %d: two runs differ" % path


@pytest.mark.parametrize("seed", range(120))
def test_random_part_call(cabi, seed):
    """One part-level entry point per draw: random l, channel counts, channel offset, grid, batch broadcast, views with
    a channel stride, accumulate or overwrite."""
    rng = np.random.default_rng(9000 + seed)
    diag = bool(rng.integers(0, 2))
    l1, l2 = int(rng.integers(0, 11)), int(rng.integers(0, 11))
    l = int(rng.integers(abs(l1 - l2), l1 + l2 + 1))
    n1 = int(rng.choice([1, 2, 3, 4, 7, 8, 16, 33, 64]))
    n2 = n1 if diag else int(rng.choice([1, 2, 3, 4, 8, 16]))
    nout = n1 if diag else n1 * n2
    offs, tail = int(rng.choice([0, 0, 3, 8])), int(rng.choice([0, 5]))
    B = int(rng.choice([1, 2, 6, 37]))
    grid = [(), (3,), (2, 2)][int(rng.integers(0, 3))]
    kind = int(rng.integers(0, 3))              # 0 forward, 1 back0, 2 back1
    accumulate = bool(rng.integers(0, 2))
    bcast = int(rng.integers(0, 4)) == 0        # an operand (not the destination) shared by the whole batch
    stride2 = int(rng.integers(0, 5)) == 0      # the destination is every second channel of a wider tensor

    def lead(b):
        return (b,) + grid

    xb = 1 if (bcast and kind != 1) else B
    yb = 1 if (bcast and kind == 1) else B
    x = U.seeded(seed * 7 + 1, *lead(xb), 2 * l1 + 1, n1)
    y = U.seeded(seed * 7 + 2, *lead(yb), 2 * l2 + 1, n2)
    r = U.seeded(seed * 7 + 3, *lead(B), 2 * l + 1, offs + nout + tail)   # product, or the incoming gradient
    full = lambda a: np.ascontiguousarray(np.broadcast_to(a, lead(B) + a.shape[-2:]))
    flat = lambda a: a.reshape((-1,) + a.shape[-2:])
    ops = (ora.DIAG_FWD, ora.DIAG_BACK0, ora.DIAG_BACK1) if diag else (ora.CG_FWD, ora.CG_BACK0, ora.CG_BACK1)
    fns = ((cabi.so3part_diagcg_fwd, cabi.so3part_diagcg_back0, cabi.so3part_diagcg_back1) if diag else
           (cabi.so3part_cg_fwd, cabi.so3part_cg_back0, cabi.so3part_cg_back1))
    dest0 = [r, U.seeded(seed * 7 + 4, *lead(B), 2 * l1 + 1, n1), U.seeded(seed * 7 + 5, *lead(B), 2 * l2 + 1, n2)][kind]

    def reference(prec):
        c = (lambda a: flat(full(a)).astype(np.complex128)) if prec == 64 else (lambda a: flat(full(a)).copy())
        d = c(dest0)
        if not accumulate:
            if kind == 0:
                d[..., offs:offs + nout] = 0      # overwrite touches the block of this triple only
            else:
                d[...] = 0
        if kind == 0:
            ora.part_op(ops[0], d, c(x), c(y), offs)
        elif kind == 1:
            ora.part_op(ops[1], c(r), d, c(y), offs)
        else:
            ora.part_op(ops[2], c(r), c(x), d, offs)
        return d

    want32, want64 = reference(32), reference(64)
    # term sums of the destination; in accumulate mode what was there before is one more term
    S = ora.part_term_sums(ops[kind], flat(full(r)), flat(full(x)), flat(full(y)), offs)
    if accumulate:
        S = S + np.abs(flat(full(dest0)))
    if stride2:
        wide = torch.zeros(dest0.shape[:-1] + (2 * dest0.shape[-1],), dtype=torch.complex64, device="cuda")
        dest = wide[..., ::2]
        dest.copy_(U.dev(dest0))
    else:
        dest = U.dev(dest0)
    dx, dy, dr = U.dev(x), U.dev(y), U.dev(r)
    args = [(dest, dx, dy), (dest, dr, dy), (dest, dr, dx)][kind]
    fns[kind](*args, offs=offs, accumulate=accumulate)
    torch.cuda.synchronize()
    tag = "seed %d kind %d diag %d (%d,%d)x(%d,%d)->%d offs %d B %d grid %s bcast %d acc %d stride2 %d path %d" % (
        seed, kind, diag, l1, n1, l2, n2, l, offs, B, grid, bcast, accumulate, stride2, cabi.last_path())
    U.assert_parity(flat(U.host(dest.contiguous())), want32, want64, S, tag)
