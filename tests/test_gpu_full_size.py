"""The benchmark configurations at their full sizes, through the C-ABI.

The CPU oracle cannot cover tens of GiB, so each configuration is checked three ways:
  * parity with the oracle on slices of the batch: the first cells, the last cells (whose offsets exceed 2^32 bytes in
    the large parts) and cells picked at random in between;
  * properties that do not depend on the size: scaling an operand by two scales the product by two bit for bit,
    reversing the batch reverses the product bit for bit;
  * the adjoint identity that ties the backward kernels to the forward one on the whole batch: with the product r itself
    as the incoming gradient, sum |r|^2 = <x, back0(r, y)> = <y, back1(r, x)> (sums in float64 on the GPU).
"""
import numpy as np
import pytest

from oracle import cg_oracle as ora
from tests import gpu_util as U

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

# name: (batch, tau_x, tau_y, maxl, diag, scale of y, also run the bit-exact properties (needs a second product))
CONFIGS = {
    "cfg1_part_1x1to1_n16_B1024": (1024, {1: 16}, {1: 16}, 1, False, 1.0, True),
    "cfg2_part_2x3to4_n32_B65536": (65536, {2: 32}, {3: 32}, 4, False, 1.0, True),
    "cfg4_vec_L4_tau16_B32768_maxl4": (32768, {l: 16 for l in range(5)}, {l: 16 for l in range(5)}, 4, False, 1.0, True),
    "cfg5_part_10x10_all_l_n8_B16384": (16384, {10: 8}, {10: 8}, -1, False, 1e-3, True),
    "cfg3_vec_diag_L6_n64_B131072": (131072, {l: 64 for l in range(7)}, {l: 64 for l in range(7)}, 6, True, 1.0, False),
}


@pytest.fixture(scope="module")
def cabi():
    assert torch.cuda.is_available()
    from gelib_amd import cabi as c
    c.lib()
    return c


def out_type(tx, ty, maxl, diag):
    tau = {}
    for l1, n1 in sorted(tx.items()):
        for l2, n2 in sorted(ty.items()):
            for l in range(abs(l1 - l2), l1 + l2 + 1):
                if maxl < 0 or l <= maxl:
                    tau[l] = tau.get(l, 0) + (n1 if diag else n1 * n2)
    return dict(sorted(tau.items()))


def parts(B, tau, seed, scale=1.0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return [torch.view_as_complex(torch.randn(B, 2 * l + 1, n, 2, device="cuda", generator=g)) * scale for l, n in tau.items()]


def dot64(a, b, chunks=16):
    """sum over the components of a * b, accumulated in float64 on the GPU, a slab of the batch at a time."""
    tot = 0.0
    n = a.shape[0]
    step = (n + chunks - 1) // chunks
    for s in range(0, n, step):
        ra = torch.view_as_real(a[s:s + step]).double()
        rb = torch.view_as_real(b[s:s + step]).double()
        tot += float((ra * rb).sum())
    return tot


@pytest.mark.parametrize("name", list(CONFIGS))
def test_full_size(cabi, name):
    B, tx, ty, maxl, diag, yscale, bitwise = CONFIGS[name]
    free, _ = torch.cuda.mem_get_info()
    tr = out_type(tx, ty, maxl, diag)
    need = 8 * B * sum((2 * l + 1) * n for l, n in tr.items()) * (2.3 if bitwise else 1.3)
    if free < need:
        pytest.skip("needs %.0f GB of free device memory" % (need / 1e9))
    xs, ys = parts(B, tx, 11), parts(B, ty, 12, yscale)
    rs = [torch.empty(B, 2 * l + 1, n, dtype=torch.complex64, device="cuda") for l, n in tr.items()]
    cabi.so3vec_fwd(rs, xs, ys, accumulate=False, diag=diag)

    # slices against the oracle
    rng = np.random.default_rng(5)
    k = 8 if sum(tr.values()) > 4096 else 32
    idx = np.unique(np.concatenate([np.arange(k), np.arange(B - k, B), rng.integers(0, B, k)]))
    tidx = torch.from_numpy(idx).cuda()
    hx = [U.host(t[tidx]) for t in xs]
    hy = [U.host(t[tidx]) for t in ys]
    O = U.VecOracle(hx, hy, maxl, diag, nthreads=8)
    O.check_fwd([U.host(t[tidx]) for t in rs], name)

    # the adjoint identity on the whole batch, the product itself as the incoming gradient
    xg = [torch.empty_like(t) for t in xs]
    yg = [torch.empty_like(t) for t in ys]
    cabi.so3vec_bwd(xg, yg, rs, xs, ys, accumulate=False, diag=diag)
    rr = sum(dot64(t, t) for t in rs)
    xx = sum(dot64(a, b) for a, b in zip(xs, xg))
    yy = sum(dot64(a, b) for a, b in zip(ys, yg))
    assert rr > 0
    assert abs(xx - rr) <= 2e-5 * rr, (name, rr, xx)
    assert abs(yy - rr) <= 2e-5 * rr, (name, rr, yy)
    # and the gradients of the slices against the oracle, every component under the rules of tests/gpu_util.py
    O.set_gradient([U.host(t[tidx]) for t in rs], nthreads=8)
    O.check_bwd([U.host(t[tidx]) for t in xg], [U.host(t[tidx]) for t in yg], name)
    del xg, yg

    if not bitwise:
        return
    r2 = [torch.empty_like(t) for t in rs]
    cabi.so3vec_fwd(r2, [2 * t for t in xs], ys, accumulate=False, diag=diag)
    for a, b in zip(rs, r2):
        assert torch.equal(torch.view_as_real(b), 2 * torch.view_as_real(a)), name
    cabi.so3vec_fwd(r2, [t.flip(0).contiguous() for t in xs], [t.flip(0).contiguous() for t in ys], accumulate=False,
                    diag=diag)
    for a, b in zip(rs, r2):
        step = max(1, B // 8)
        for s in range(0, B, step):     # a slab at a time: the flipped copy of a whole part would double the footprint
            hi = min(B, s + step)
            assert torch.equal(b[s:hi], a[B - hi:B - s].flip(0)), name


@pytest.mark.parametrize("case", [(1024, 1, 16, 1, 16, 1), (65536, 2, 32, 3, 32, 4)])
def test_single_triple_configs(cabi, case):
    """Configurations 1 and 2 exactly as listed: ONE (l1, l2, l) triple at full batch through the part-level entry
    points (the reference's SO3part operator: add_CGproduct, add_CGproduct_back0, add_CGproduct_back1), and both
    gradients once more from one pass over g (what the Python operator runs when no operand is broadcast).  Slices of
    the batch are checked against the oracle's loops for the single triple."""
    B, l1, n1, l2, n2, l = case
    (x,), (y,) = parts(B, {l1: n1}, 21), parts(B, {l2: n2}, 22)
    (g,) = parts(B, {l: n1 * n2}, 23)
    r = torch.full((B, 2 * l + 1, n1 * n2), 3.0 - 1j, dtype=torch.complex64, device="cuda")
    cabi.so3part_cg_fwd(r, x, y, 0, accumulate=False)
    xg0 = torch.full_like(x, 5.0)
    yg0 = torch.full_like(y, 5.0)
    cabi.so3part_cg_back0(xg0, g, y, 0, accumulate=False)
    cabi.so3part_cg_back1(yg0, g, x, 0, accumulate=False)
    xg1, yg1 = torch.full_like(x, 7.0), torch.full_like(y, 7.0)
    cabi.so3vec_bwd([xg1], [yg1], [g], [x], [y], accumulate=False)
    torch.cuda.synchronize()
    rng = np.random.default_rng(6)
    k = 16
    idx = np.unique(np.concatenate([np.arange(k), np.arange(B - k, B), rng.integers(0, B, k)]))
    tidx = torch.from_numpy(idx).cuda()
    hx, hy, hg = U.host(x[tidx]), U.host(y[tidx]), U.host(g[tidx])
    r32 = ora.cg_fwd(hx, hy, l)
    r64 = ora.cg_fwd(*U.c128([hx, hy]), l)
    xg32, yg32 = ora.cg_bwd(hg, hx, hy)
    xg64, yg64 = ora.cg_bwd(*U.c128([hg, hx, hy]))
    Sr, Sx, Sy = ora.cg_term_sums(hg, hx, hy, l)
    what = "triple (%d,%d,%d) n %dx%d B %d" % (l1, l2, l, n1, n2, B)
    rep = U.assert_parity(U.host(r[tidx]), r32, r64, Sr, "fwd " + what)
    assert rep["outside_gate"] * rep["components"] <= 1 + 1e-7 * rep["components"], rep
    for got_x, got_y, tag in ((xg0, yg0, "back0/back1"), (xg1, yg1, "one pass")):
        U.assert_parity(U.host(got_x[tidx]), xg32, xg64, Sx, "xg %s %s" % (tag, what))
        U.assert_parity(U.host(got_y[tidx]), yg32, yg64, Sy, "yg %s %s" % (tag, what))
