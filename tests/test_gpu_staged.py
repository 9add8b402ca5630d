"""GPU parity of the any-l ("staged") kernels: operand l above 4, where the unrolled small-l kernels do not apply.

Each case checks the kernel family that ran (gelib_hip_last_path() == 3) and compares with the CPU oracle in
float32 and float64, as the other GPU tests do.  One of the two backward forms adds partial sums into LDS images with
float atomics, so its last bits can differ from run to run; the parity rules of tests/gpu_util.py hold for any order.
"""
import numpy as np
import pytest

from oracle import cg_oracle as ora
from tests import gpu_util as U

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

STAGED = 3


@pytest.fixture(scope="module", params=["striped", "pairwise", "triplewise"])
def cabi(request):
    """The three backward forms of the family: one gradient per launch with sums in registers; both gradients in
    one launch, one (x part, y part) pair at a time, contracting over l first; and both gradients in one launch,
    one triple at a time.  Each is forced wherever its conditions hold.  By itself the library uses the first only: the
    other two add partial sums with LDS float atomics and run on request ("staged_bwd_atomic")."""
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from gelib_amd import cabi as c
    c.lib()
    c.set_option("force_generic", 0)
    c.set_option("diag6", 0)   # the lane-per-channel Diag kernels would take some of these cases first
    c.set_option("onepair", 0) # and the single-pair backward kernels others
    c.set_option("onepair_mfma", 0)
    c.set_option("onepair_mfma_fwd", 0)
    c.set_option("unrolled_bwd_l6", 0)   # the unrolled backward kernel for operands up to l = 6 would take some too
    c.set_option("unrolled_fwd_l6", 0)   # ... and so would the forward kernel for operands up to l = 6
    c.set_option("pairwise_bwd", 0)
    c.set_option("staged_bwd_stripes", 1 if request.param == "striped" else 0)
    c.set_option("staged_bwd_atomic", 1)   # the other two forms (and what the striped one leaves) add with LDS float atomics
    c.set_option("staged_bwd_pairs", int(request.param == "pairwise"))
    yield c
    c.set_option("diag6", 1)
    c.set_option("onepair", 1)
    c.set_option("onepair_mfma", 1)
    c.set_option("onepair_mfma_fwd", 1)
    c.set_option("unrolled_bwd_l6", 1)
    c.set_option("unrolled_fwd_l6", 1)
    c.set_option("pairwise_bwd", 1)
    c.set_option("staged_bwd_threads", 0)
    c.set_option("staged_bwd_stripes", 1)
    c.set_option("staged_bwd_atomic", 0)
    c.set_option("staged_bwd_pairs", 0)


def c128(L):
    return [a.astype(np.complex128) for a in L]


def run_vec(cabi, B, tx, ty, maxl, diag, seed, expect_bwd=STAGED):
    xs = [U.seeded(seed + l, B, 2 * l + 1, n) for l, n in sorted(tx.items())]
    ys = [U.seeded(seed + 50 + l, B, 2 * l + 1, n) for l, n in sorted(ty.items())]
    O = U.VecOracle(xs, ys, maxl, diag, gseed=seed + 100)
    r32, gs = O.r32, O.gs
    dxs, dys, dgs = [U.dev(a) for a in xs], [U.dev(a) for a in ys], [U.dev(a) for a in gs]
    drs = [torch.full(p.shape, 7.0 + 1j, dtype=torch.complex64, device="cuda") for p in r32]
    cabi.so3vec_fwd(drs, dxs, dys, accumulate=False, diag=diag)
    assert cabi.last_path() == STAGED
    dxg = [torch.full(a.shape, 3.0 - 2j, dtype=torch.complex64, device="cuda") for a in xs]
    dyg = [torch.full(a.shape, 3.0 - 2j, dtype=torch.complex64, device="cuda") for a in ys]
    cabi.so3vec_bwd(dxg, dyg, dgs, dxs, dys, accumulate=False, diag=diag)
    assert cabi.last_path() == expect_bwd
    torch.cuda.synchronize()
    tag = "B%d %s x %s maxl %d diag %d" % (B, tx, ty, maxl, diag)
    O.check_fwd([U.host(a) for a in drs], tag)
    O.check_bwd([U.host(a) for a in dxg], [U.host(a) for a in dyg], tag)
    # accumulate mode adds on top of what is there; one gradient at a time
    drs2 = [a.clone() for a in drs]
    cabi.so3vec_fwd(drs2, dxs, dys, accumulate=True, diag=diag)
    dxg2 = [a.clone() for a in dxg]
    dyg2 = [a.clone() for a in dyg]
    cabi.so3vec_bwd(dxg2, None, dgs, dxs, dys, accumulate=True, diag=diag)
    cabi.so3vec_bwd(None, dyg2, dgs, dxs, dys, accumulate=True, diag=diag)
    torch.cuda.synchronize()
    for a, b in zip(drs2, drs):
        assert U.gate_excess(U.host(a), 2 * U.host(b)) <= 1.0
    O.check_bwd_onto([U.host(a) for a in dxg2], [U.host(a) for a in dyg2], [U.host(a) for a in dxg],
                     [U.host(a) for a in dyg], tag + " accumulated")


VEC_CASES = [
    # (B, tau_x, tau_y, maxl)
    (5, {l: 8 for l in range(7)}, {l: 8 for l in range(7)}, 6),    # the Diag L=6 benchmark type, small
    (3, {10: 8}, {10: 8}, -1),                                       # l up to 20: g passes the registers in two windows
    (7, {5: 4, 6: 2}, {0: 2, 7: 4}, -1),                             # l up to 13: 27 rows, the 32-row variant
    (70, {5: 1}, {6: 1}, -1),                                        # one channel: many cells share a run
    (2, {6: 16}, {5: 16}, 8),                                        # 256 slots per cell: several runs per cell
    (3, {5: 2, 6: 4}, {5: 4, 6: 8}, 7),                              # channel counts differ between parts
    (2, {12: 2}, {3: 4}, -1),                                        # own l = 12: 25 rows, the 32-row variant
    (3, {5: 4, 9: 4}, {5: 4}, 3),                                    # x part l = 9 feeds nothing (l >= 4 is cut): zero gradient
]


@pytest.mark.parametrize("case", VEC_CASES)
@pytest.mark.parametrize("diag", [False, True])
def test_vec(cabi, case, diag):
    B, tx, ty, maxl = case
    if diag:
        n = tx[min(tx)]
        tx, ty = {l: n for l in tx}, {l: n for l in ty}
    run_vec(cabi, B, tx, ty, maxl, diag, seed=500)


def test_diag_with_more_channels_than_a_wave(cabi):
    # 128 and 96 channels: two runs of 64 lane slots per cell, each flushed on its own
    run_vec(cabi, 3, {5: 128}, {5: 128}, 6, True, seed=520)
    run_vec(cabi, 3, {5: 96, 6: 96}, {5: 96}, 7, True, seed=521)


@pytest.mark.parametrize("threads", [256, 512, 1024])
def test_backward_block_widths(cabi, threads):
    cabi.set_option("staged_bwd_threads", threads)
    try:
        run_vec(cabi, 6, {l: 4 for l in range(6)}, {l: 4 for l in range(6)}, 5, False, seed=600)
        run_vec(cabi, 6, {l: 4 for l in range(6)}, {l: 4 for l in range(6)}, 5, True, seed=601)
    finally:
        cabi.set_option("staged_bwd_threads", 0)


@pytest.mark.parametrize("tile", [1, 2, 4])
def test_forward_tile_widths(cabi, tile):
    cabi.set_option("staged_fwd_tile", tile)
    try:
        run_vec(cabi, 37, {5: 8, 6: 8}, {5: 8, 6: 8}, 9, False, seed=650)
        run_vec(cabi, 37, {5: 8, 6: 8}, {5: 8, 6: 8}, 9, True, seed=651)
        run_vec(cabi, 3, {6: 64}, {6: 64}, 6, True, seed=652)
    finally:
        cabi.set_option("staged_fwd_tile", 0)


def test_channel_counts_that_are_not_powers_of_two(cabi):
    # the forward kernel takes any channel count; the backward kernels round the counts up to powers of two for their
    # lane layout and idle the lanes beyond the real channels
    run_vec(cabi, 4, {5: 3, 6: 5}, {5: 6, 1: 7}, -1, False, seed=700)
    run_vec(cabi, 4, {5: 3, 6: 3}, {5: 3, 1: 3}, -1, True, seed=701)
    run_vec(cabi, 9, {6: 12}, {5: 12}, 7, False, seed=702)          # 12 x 12 -> 16 x 16 lane slots, several runs per cell
    run_vec(cabi, 40, {7: 1}, {5: 3}, -1, False, seed=703)          # 3 -> 4 lane slots per cell, 16 cells per run


@pytest.mark.parametrize("offs", [3, 4])   # odd: one channel per lane; multiple of 4: four adjacent channels per lane
@pytest.mark.parametrize("diag", [False, True])
def test_part_level_with_offset(cabi, diag, offs):
    B, l1, l2, l, n1, n2, extra = 9, 6, 5, 7, 4, (4 if diag else 8), 4
    nout = n1 if diag else n1 * n2
    x, y = U.seeded(1, B, 2 * l1 + 1, n1), U.seeded(2, B, 2 * l2 + 1, n2)
    g = U.seeded(3, B, 2 * l + 1, offs + nout + extra)
    fwd = cabi.so3part_diagcg_fwd if diag else cabi.so3part_cg_fwd
    b0 = cabi.so3part_diagcg_back0 if diag else cabi.so3part_cg_back0
    b1 = cabi.so3part_diagcg_back1 if diag else cabi.so3part_cg_back1
    r0 = U.seeded(4, B, 2 * l + 1, offs + nout + extra)
    op_f, op_0, op_1 = (ora.DIAG_FWD, ora.DIAG_BACK0, ora.DIAG_BACK1) if diag else (ora.CG_FWD, ora.CG_BACK0, ora.CG_BACK1)
    want, want64 = r0.copy(), r0.astype(np.complex128)
    ora.part_op(op_f, want, x, y, offs)            # the reference's add into what is there
    ora.part_op(op_f, want64, x.astype(np.complex128), y.astype(np.complex128), offs)
    Sr = ora.part_term_sums(op_f, r0, x, y, offs) + np.abs(r0)
    dr = U.dev(r0)
    fwd(dr, U.dev(x), U.dev(y), offs, accumulate=True)
    assert cabi.last_path() == STAGED
    torch.cuda.synchronize()
    U.assert_parity(U.host(dr), want, want64, Sr, "part fwd onto r0")
    # outside the block nothing moves
    assert np.array_equal(U.host(dr)[:, :, :offs], r0[:, :, :offs])
    assert np.array_equal(U.host(dr)[:, :, offs + nout:], r0[:, :, offs + nout:])
    gblock = np.ascontiguousarray(g[:, :, offs:offs + nout])
    xg32, yg32 = ora.cg_bwd(gblock, x, y, diag)
    xg64, yg64 = ora.cg_bwd(gblock.astype(np.complex128), x.astype(np.complex128), y.astype(np.complex128), diag)
    dxg = torch.full(x.shape, 5.0 + 5j, dtype=torch.complex64, device="cuda")
    dyg = torch.full(y.shape, 5.0 + 5j, dtype=torch.complex64, device="cuda")
    b0(dxg, U.dev(g), U.dev(y), offs, accumulate=False)
    assert cabi.last_path() == STAGED
    b1(dyg, U.dev(g), U.dev(x), offs, accumulate=False)
    assert cabi.last_path() == STAGED
    torch.cuda.synchronize()
    U.assert_parity(U.host(dxg), xg32, xg64, ora.part_term_sums(op_0, g, x, y, offs), "part back0")
    U.assert_parity(U.host(dyg), yg32, yg64, ora.part_term_sums(op_1, g, x, y, offs), "part back1")


def test_broadcast_operand_and_grid(cabi):
    # y is shared by the whole batch (stride 0) and the cells form a (batch, grid) array
    B, G0, l1, l2, l, n = 3, 4, 5, 5, 6, 4
    x = U.seeded(11, B, G0, 2 * l1 + 1, n)
    y = U.seeded(12, 1, 1, 2 * l2 + 1, n)
    want = ora.cg_fwd(x.reshape(B * G0, 2 * l1 + 1, n), np.broadcast_to(y, (B, G0) + y.shape[2:]).reshape(B * G0, 2 * l2 + 1, n), l)
    dr = torch.zeros(B, G0, 2 * l + 1, n * n, dtype=torch.complex64, device="cuda")
    dy = U.dev(y).expand(B, G0, 2 * l2 + 1, n)
    cabi.so3part_cg_fwd(dr, U.dev(x), dy, 0, accumulate=False)
    assert cabi.last_path() == STAGED
    torch.cuda.synchronize()
    assert U.gate_excess(U.host(dr).reshape(want.shape), want) <= 1.0
