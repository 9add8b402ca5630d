"""GPU parity of the lane-per-channel Diag kernels (operand l up to 6, more than 32 channels, product l up to 6):
gelib_hip_last_path() == 4, results against the CPU oracle in float32 and float64."""
import numpy as np
import pytest

from oracle import cg_oracle as ora
from tests import gpu_util as U

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

DIAG6 = 4


@pytest.fixture(scope="module")
def cabi():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from gelib_amd import cabi as c
    c.lib()
    c.set_option("force_generic", 0)
    c.set_option("diag6", 1)
    return c


def c128(L):
    return [a.astype(np.complex128) for a in L]


CASES = [
    # (B, tau_x, tau_y, maxl)
    (5, {l: 64 for l in range(7)}, {l: 64 for l in range(7)}, 6),      # the benchmark type, small batch
    (3, {l: 96 for l in range(6)}, {l: 96 for l in range(6)}, 5),      # two channel groups, the second half empty
    (4, {0: 40, 5: 40}, {1: 40, 6: 40}, 6),                            # parts missing, 40 of 64 lanes live
    (2, {6: 64}, {6: 64}, 6),                                          # one pair, l from 0 to 6 of 0..12
    (3, {2: 64, 6: 64}, {3: 64, 5: 64}, 4),                            # capped below the largest operand l
    (1, {l: 200 for l in range(7)}, {l: 200 for l in range(7)}, 6),    # four groups, one cell
    (70, {5: 33}, {4: 33}, 6),                                         # 33 channels: one group, 31 lanes idle
    (37, {l: 16 for l in range(5)}, {l: 16 for l in range(5)}, 4),     # four cells per wave, the last wave one cell
    (130, {0: 1, 3: 1}, {2: 1, 3: 1}, 6),                              # one channel: 64 cells per wave
    (9, {l: 24 for l in range(7)}, {l: 24 for l in range(7)}, 6),      # two cells per wave, 8 lanes of each idle
    (5, {1: 32, 6: 32}, {6: 32}, 5),                                   # exactly half a wave per cell
    (3, {1: 64, 4: 64}, {l: 64 for l in range(7)}, 6),                 # every part of y, parts of x missing
    (2, {l: 64 for l in range(7)}, {l: 64 for l in range(7)}, 3),      # every part of y, product capped low
    # operands up to l = 2 (and backward up to l = 4): a wave, not a block, per cell and channel group
    (70, {0: 5, 1: 5}, {0: 5, 1: 5}, -1),                              # eight cells per wave, three lanes of each idle
    (9, {l: 96 for l in range(3)}, {l: 96 for l in range(3)}, -1),     # two channel groups, product up to l = 4
    (33, {1: 64}, {0: 64, 2: 64}, 2),                                  # parts missing, capped
    (6, {l: 64 for l in range(5)}, {l: 64 for l in range(5)}, 4),      # operands up to l = 4, one cell per wave
    (7, {2: 40, 4: 40}, {1: 40, 3: 40}, 6),                            # ... parts missing, product up to l = 6
]


@pytest.mark.parametrize("B,tx,ty,maxl", CASES)
def test_diag6_vec(cabi, B, tx, ty, maxl):
    seed = 900 + B
    xs = [U.seeded(seed + l, B, 2 * l + 1, n) for l, n in sorted(tx.items())]
    ys = [U.seeded(seed + 50 + l, B, 2 * l + 1, n) for l, n in sorted(ty.items())]
    O = U.VecOracle(xs, ys, maxl, True, gseed=seed + 100)
    r32, gs = O.r32, O.gs
    dxs, dys, dgs = [U.dev(a) for a in xs], [U.dev(a) for a in ys], [U.dev(a) for a in gs]
    drs = [torch.full(p.shape, 7.0 + 1j, dtype=torch.complex64, device="cuda") for p in r32]
    cabi.so3vec_fwd(drs, dxs, dys, accumulate=False, diag=True)
    assert cabi.last_path() == DIAG6
    dxg = [torch.full(a.shape, 3.0 - 2j, dtype=torch.complex64, device="cuda") for a in xs]
    dyg = [torch.full(a.shape, 3.0 - 2j, dtype=torch.complex64, device="cuda") for a in ys]
    cabi.so3vec_bwd(dxg, dyg, dgs, dxs, dys, accumulate=False, diag=True)
    assert cabi.last_path() == DIAG6
    torch.cuda.synchronize()
    tag = "B%d %s x %s maxl %d" % (B, tx, ty, maxl)
    O.check_fwd([U.host(a) for a in drs], tag)
    O.check_bwd([U.host(a) for a in dxg], [U.host(a) for a in dyg], tag)
    # accumulate mode adds on top of what is there
    drs2 = [a.clone() for a in drs]
    cabi.so3vec_fwd(drs2, dxs, dys, accumulate=True, diag=True)
    dxg2, dyg2 = [a.clone() for a in dxg], [a.clone() for a in dyg]
    cabi.so3vec_bwd(dxg2, dyg2, dgs, dxs, dys, accumulate=True, diag=True)
    assert cabi.last_path() == DIAG6
    torch.cuda.synchronize()
    for a, b in zip(drs2, drs):
        assert U.gate_excess(U.host(a), 2 * U.host(b)) <= 1.0
    O.check_bwd_onto([U.host(a) for a in dxg2], [U.host(a) for a in dyg2], [U.host(a) for a in dxg],
                     [U.host(a) for a in dyg], tag + " accumulated")
    # one gradient per call: the same kernel with the other one switched off, bit for bit the same sums
    dxg3 = [torch.full_like(a, 9.0) for a in dxg]
    dyg3 = [torch.full_like(a, 9.0) for a in dyg]
    cabi.so3vec_bwd(dxg3, None, dgs, dxs, dys, accumulate=False, diag=True)
    assert cabi.last_path() == DIAG6
    cabi.so3vec_bwd(None, dyg3, dgs, dxs, dys, accumulate=False, diag=True)
    assert cabi.last_path() == DIAG6
    for a, b in zip(dxg3 + dyg3, dxg + dyg):
        assert torch.equal(torch.view_as_real(a), torch.view_as_real(b))


def test_diag6_declines_what_it_cannot_do(cabi):
    # a product above l = 6 is shared with the other families; the gradient of an operand shared by the batch is formed
    # per cell by these kernels and summed over the batch by the library
    x = [U.dev(U.seeded(1, 1, 13, 64))]
    y = [U.dev(U.seeded(2, 4, 13, 64))]
    r = [torch.zeros(4, 2 * l + 1, 64, dtype=torch.complex64, device="cuda") for l in range(13)]
    cabi.so3vec_fwd(r, x, y, accumulate=False, diag=True)
    assert cabi.last_path() == DIAG6          # product l up to 12: split at l = 6
    want = ora.vec_fwd([U.host(x[0])], [U.host(y[0])], -1, True)
    for a, b in zip(r, want):
        assert U.gate_excess(U.host(a), b) <= 1.0
    r6 = r[:7]
    cabi.so3vec_fwd(r6, x, y, accumulate=False, diag=True)
    assert cabi.last_path() == DIAG6          # a broadcast x is fine going forward
    for a, b in zip(r6, want[:7]):
        assert U.gate_excess(U.host(a), b) <= 1.0
    xg, yg = [torch.zeros_like(x[0])], [torch.zeros_like(y[0])]
    cabi.so3vec_bwd(xg, yg, r6, x, y, accumulate=False, diag=True)
    assert cabi.last_path() == DIAG6          # one gradient per cell from these kernels, then the sum over the batch
    torch.cuda.synchronize()
    O = U.VecOracle([U.host(x[0])], [U.host(y[0])], 6, True, gs=[U.host(a) for a in r6])
    O.check_bwd([U.host(xg[0])], [U.host(yg[0])], "x shared by the batch")
    # a broadcast operand with several cells per wave
    x8 = [U.dev(U.seeded(3, 1, 11, 8))]
    y8 = [U.dev(U.seeded(4, 21, 11, 8))]
    r8 = [torch.zeros(21, 2 * l + 1, 8, dtype=torch.complex64, device="cuda") for l in range(7)]
    cabi.so3vec_fwd(r8, x8, y8, accumulate=False, diag=True)
    assert cabi.last_path() == DIAG6
    want8 = ora.vec_fwd([U.host(x8[0])], [U.host(y8[0])], 6, True)
    for a, b in zip(r8, want8):
        assert U.gate_excess(U.host(a), b) <= 1.0


@pytest.mark.parametrize("l8", [1, 2, 0])
@pytest.mark.parametrize("B,tau,maxl", [(5, {l: 64 for l in range(5)}, -1), (3, {l: 16 for l in range(7)}, -1),
                                        (4, {2: 40, 6: 40}, 9), (6, {l: 16 for l in range(5)}, -1),
                                        (3, {1: 96, 4: 96}, 7), (70, {3: 5, 4: 5}, -1),
                                        (2, {l: 64 for l in range(7)}, -1), (3, {3: 70, 5: 70, 6: 70}, -1)])
def test_diag_product_above_l6(cabi, B, tau, maxl, l8):
    """A Diag product whose l reaches above 6.  Operands up to l = 4 (product up to l = 8): one launch of the
    lane-per-channel kernels built for that case (forward with l8 = 1, backward too with l8 = 2).  Otherwise, or with those
    kernels switched off: the triples
    up to l = 6 run on the lane-per-channel kernels, the rest (l = 7..12) on a second launch of that family built for those
    l (l8 = 0 here also switches that launch off) or on the other families, the gradients of the
    second part added on top of the first."""
    cabi.set_option("diag6_l8", l8)
    cabi.set_option("diag6_hi", 1 if l8 else 0)
    try:
        _above_l6(cabi, B, tau, maxl)
    finally:
        cabi.set_option("diag6_l8", 1)
        cabi.set_option("diag6_hi", 1)


def _above_l6(cabi, B, tau, maxl):
    xs = [U.seeded(40 + l, B, 2 * l + 1, n) for l, n in sorted(tau.items())]
    ys = [U.seeded(60 + l, B, 2 * l + 1, n) for l, n in sorted(tau.items())]
    O = U.VecOracle(xs, ys, maxl, True, gseed=80)
    r32, gs = O.r32, O.gs
    assert max((p.shape[1] - 1) // 2 for p in r32) > 6
    dxs, dys, dgs = [U.dev(a) for a in xs], [U.dev(a) for a in ys], [U.dev(a) for a in gs]
    for accumulate in (False, True):
        start = 5.0 - 1j if accumulate else 7.0 + 1j
        drs = [torch.full(p.shape, start, dtype=torch.complex64, device="cuda") for p in r32]
        cabi.so3vec_fwd(drs, dxs, dys, accumulate=accumulate, diag=True)
        assert cabi.last_path() == DIAG6
        dxg = [torch.full(a.shape, start, dtype=torch.complex64, device="cuda") for a in xs]
        dyg = [torch.full(a.shape, start, dtype=torch.complex64, device="cuda") for a in ys]
        cabi.so3vec_bwd(dxg, dyg, dgs, dxs, dys, accumulate=accumulate, diag=True)
        assert cabi.last_path() == DIAG6
        torch.cuda.synchronize()
        hr, hxg, hyg = [U.host(a) for a in drs], [U.host(a) for a in dxg], [U.host(a) for a in dyg]
        if accumulate:
            full = lambda parts: [np.full(p.shape, start, dtype=np.complex64) for p in parts]
            O.check_fwd_onto(hr, full(r32), "split Diag product onto a constant")
            O.check_bwd_onto(hxg, hyg, full(xs), full(ys), "split Diag gradients onto a constant")
        else:
            O.check_fwd(hr, "split Diag product")
            O.check_bwd(hxg, hyg, "split Diag gradients")


ONE_CHANNEL = [
    # (B, channels of the wide operand, l of the wide parts, l of the one-channel parts, maxl, narrow side)
    (37, 16, range(5), range(3), 4, "y"),        # features x single-channel harmonics, four cells per wave
    (37, 16, range(5), range(3), -1, "y"),       # uncapped: l up to 6
    (9, 64, range(4), range(4), 6, "y"),         # one cell per wave
    (11, 40, [0, 2, 5], [1, 6], 6, "x"),         # the first operand is the narrow one; 24 lanes idle
    (70, 5, [3, 4], [2], 6, "x"),                # eight cells per wave, three lanes of each idle
    (5, 64, range(7), range(7), 6, "y"),         # every part of y: the kernel with fixed sets of l2 per wave
    (3, 16, range(5), range(5), -1, "y"),        # product up to l = 8: split at l = 6 (or the l <= 8 kernels forward)
    (37, 16, range(3), range(2), -1, "y"),       # wide parts up to l = 2: the kernels that give a wave a cell
    (9, 64, range(3), range(3), 4, "x"),
]


@pytest.mark.parametrize("B,n,lw,ln,maxl,narrow", ONE_CHANNEL)
def test_cgproduct_with_a_one_channel_operand(cabi, B, n, lw, ln, maxl, narrow):
    """CGproduct in which every part of one operand has ONE channel (features times single-channel spherical harmonics,
    the usual use of add_spharm's output): the lane-per-channel kernels take it as the Diag product with that channel
    repeated -- every lane reads the one channel, its gradient is summed over the lanes of a cell.  Against the oracle's
    CGproduct loops."""
    seed = 4000 + B
    wide = [U.seeded(seed + l, B, 2 * l + 1, n) for l in lw]
    thin = [U.seeded(seed + 50 + l, B, 2 * l + 1, 1) for l in ln]
    xs, ys = (thin, wide) if narrow == "x" else (wide, thin)
    O = U.VecOracle(xs, ys, maxl, False, gseed=seed + 100)
    dxs, dys, dgs = [U.dev(a) for a in xs], [U.dev(a) for a in ys], [U.dev(a) for a in O.gs]
    drs = [torch.full(p.shape, 7.0 + 1j, dtype=torch.complex64, device="cuda") for p in O.r32]
    cabi.so3vec_fwd(drs, dxs, dys, accumulate=False)
    assert cabi.last_path() == DIAG6
    dxg = [torch.full(a.shape, 3.0 - 2j, dtype=torch.complex64, device="cuda") for a in xs]
    dyg = [torch.full(a.shape, 3.0 - 2j, dtype=torch.complex64, device="cuda") for a in ys]
    cabi.so3vec_bwd(dxg, dyg, dgs, dxs, dys, accumulate=False)
    assert cabi.last_path() == DIAG6
    torch.cuda.synchronize()
    tag = "B%d n%d %s x %s maxl %d narrow %s" % (B, n, list(lw), list(ln), maxl, narrow)
    O.check_fwd([U.host(a) for a in drs], tag)
    O.check_bwd([U.host(a) for a in dxg], [U.host(a) for a in dyg], tag)
    # accumulate mode, and one gradient per call (bit for bit the same sums)
    dxg2, dyg2 = [a.clone() for a in dxg], [a.clone() for a in dyg]
    cabi.so3vec_bwd(dxg2, dyg2, dgs, dxs, dys, accumulate=True)
    torch.cuda.synchronize()
    O.check_bwd_onto([U.host(a) for a in dxg2], [U.host(a) for a in dyg2], [U.host(a) for a in dxg],
                     [U.host(a) for a in dyg], tag + " accumulated")
    dxg3, dyg3 = [torch.full_like(a, 9.0) for a in dxg], [torch.full_like(a, 9.0) for a in dyg]
    cabi.so3vec_bwd(dxg3, None, dgs, dxs, dys, accumulate=False)
    cabi.so3vec_bwd(None, dyg3, dgs, dxs, dys, accumulate=False)
    if maxl <= 6 and max(list(lw)) + max(list(ln)) <= 6 or maxl in range(0, 7):
        for a, b in zip(dxg3 + dyg3, dxg + dyg):
            assert torch.equal(torch.view_as_real(a), torch.view_as_real(b))
    # the general kernels give the same to rounding
    cabi.set_option("diag6_one_channel", 0)
    try:
        cabi.so3vec_bwd(dxg3, dyg3, dgs, dxs, dys, accumulate=False)
        assert cabi.last_path() != DIAG6
        torch.cuda.synchronize()
        O.check_bwd([U.host(a) for a in dxg3], [U.host(a) for a in dyg3], tag + " general kernels")
    finally:
        cabi.set_option("diag6_one_channel", 1)


def test_one_channel_operand_with_many_channels_on_the_other_side(cabi):
    # more than 64 channels: forward here (any count), the gradient of the one-channel operand on the other families
    B, n = 4, 96
    xs = [U.seeded(10 + l, B, 2 * l + 1, n) for l in range(3)]
    ys = [U.seeded(20 + l, B, 2 * l + 1, 1) for l in range(3)]
    O = U.VecOracle(xs, ys, 4, False, gseed=77)
    dxs, dys, dgs = [U.dev(a) for a in xs], [U.dev(a) for a in ys], [U.dev(a) for a in O.gs]
    drs = [torch.empty(p.shape, dtype=torch.complex64, device="cuda") for p in O.r32]
    cabi.so3vec_fwd(drs, dxs, dys, accumulate=False)
    assert cabi.last_path() == DIAG6
    dxg, dyg = [torch.empty_like(a) for a in dxs], [torch.empty_like(a) for a in dys]
    cabi.so3vec_bwd(dxg, dyg, dgs, dxs, dys, accumulate=False)
    assert cabi.last_path() != DIAG6
    cabi.so3vec_bwd(dxg, None, dgs, dxs, dys, accumulate=False)
    assert cabi.last_path() == DIAG6      # the wide operand's gradient alone needs no sum over lanes
    torch.cuda.synchronize()
    O.check_fwd([U.host(a) for a in drs], "n 96")
    O.check_bwd([U.host(a) for a in dxg], [U.host(a) for a in dyg], "n 96")


@pytest.mark.parametrize("B,ls,maxl", [(70, range(5), 4), (33, range(7), -1), (5, (1, 3, 6), 9), (130, range(3), -1)])
def test_cgproduct_of_one_channel_vectors_goes_forward_on_the_diag_kernels(cabi, B, ls, maxl):
    """One channel in every part of both operands (products of spherical harmonics, say): block channel 0 * 1 + 0, the
    Diag product of one channel.  Forward it runs on the lane-per-channel kernels, a cell per lane (split at l = 6 when
    the product reaches higher); the gradients stay with the other families."""
    xs = [U.seeded(900 + l, B, 2 * l + 1, 1) for l in ls]
    ys = [U.seeded(950 + l, B, 2 * l + 1, 1) for l in ls]
    O = U.VecOracle(xs, ys, maxl, False, gseed=990)
    dxs, dys, dgs = [U.dev(a) for a in xs], [U.dev(a) for a in ys], [U.dev(a) for a in O.gs]
    drs = [torch.full(p.shape, 7.0 + 1j, dtype=torch.complex64, device="cuda") for p in O.r32]
    cabi.so3vec_fwd(drs, dxs, dys, accumulate=False)
    assert cabi.last_path() == DIAG6
    torch.cuda.synchronize()
    O.check_fwd([U.host(a) for a in drs], "one channel on both sides, forward")
    start = [U.seeded(970 + k, *p.shape) for k, p in enumerate(O.r32)]
    drs2 = [U.dev(a) for a in start]
    cabi.so3vec_fwd(drs2, dxs, dys, accumulate=True)
    torch.cuda.synchronize()
    O.check_fwd_onto([U.host(a) for a in drs2], start, "one channel on both sides, forward onto")
    dxg = [torch.full(a.shape, 3.0 - 2j, dtype=torch.complex64, device="cuda") for a in xs]
    dyg = [torch.full(a.shape, 3.0 - 2j, dtype=torch.complex64, device="cuda") for a in ys]
    cabi.so3vec_bwd(dxg, dyg, dgs, dxs, dys, accumulate=False)
    assert cabi.last_path() != DIAG6
    torch.cuda.synchronize()
    O.check_bwd([U.host(a) for a in dxg], [U.host(a) for a in dyg], "one channel on both sides, backward")
