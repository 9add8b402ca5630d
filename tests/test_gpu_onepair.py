"""GPU parity of the kernels for products of ONE x part with ONE y part of large l (l1 + l2 <= 21, at most 64 channel
slots per cell, or one of the channel counts the matrix-core kernels are built for): gelib_hip_last_path() == 5,
gradients (and, on the matrix cores, the product itself) against the CPU oracle in float32 and float64."""
import numpy as np
import pytest

from oracle import cg_oracle as ora
from tests import gpu_util as U

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

ONEPAIR = 5


@pytest.fixture(scope="module")
def cabi():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from gelib_amd import cabi as c
    c.lib()
    c.set_option("force_generic", 0)
    c.set_option("onepair", 1)
    # operands up to l = 6 with power-of-two channel counts would go to the unrolled kernels (two launches, l <= 6 and
    # l = 7..12), which are faster there; this file is about the single-pair family
    c.set_option("unrolled_bwd_l6_split", 0)
    yield c
    c.set_option("unrolled_bwd_l6_split", 1)


def c128(L):
    return [a.astype(np.complex128) for a in L]


CASES = [
    # (B, l1, n1, l2, n2, maxl, diag)
    (9, 10, 8, 10, 8, -1, False),    # the benchmark pair: 64 slots, every l from 0 to 20
    (7, 5, 3, 6, 5, -1, False),      # 3 x 5 channels padded to 4 x 8 slots, two cells per wave, odd batch
    (5, 10, 2, 11, 4, -1, False),    # l1 + l2 = 21: 44 rows of sums, 21 values of l starting at 1
    (6, 8, 8, 8, 8, 9, False),       # product capped below l1 + l2
    (11, 7, 20, 7, 20, -1, True),    # Diag, 20 channels padded to 32: two cells per wave
    (3, 9, 64, 6, 64, -1, True),     # Diag, a full wave per cell
    (70, 6, 1, 5, 1, -1, False),     # one channel pair: 64 cells per wave
    # 8 x 8 channels: the contraction over l runs on the matrix cores
    (4, 12, 8, 9, 8, -1, False),     # l1 != l2: l from 3 to 21, 19 values
    (3, 3, 8, 15, 8, -1, False),     # few rows of x, many of y: most columns of the matrix instructions idle
    (5, 15, 8, 4, 8, -1, False),     # 31 rows of x: every column but the spare one in use
    (7, 10, 8, 10, 8, 14, False),    # capped: m runs to 14 only, rows of the y-gradient end their journey early
    (2, 7, 8, 7, 8, 3, False),       # four values of l
    (33, 10, 8, 1, 8, -1, False),    # three values of l: left to the kernel that keeps its sums in LDS
    # other channel counts on the matrix cores
    (9, 10, 4, 10, 4, -1, False),    # 16 channels: one matrix tile, the x-gradient is added over the halves of the wave
    (5, 8, 4, 9, 4, -1, False),      # the same with l1 != l2
    (6, 10, 8, 10, 16, -1, False),   # 128 channels: two waves per cell, a lane holds half a row of j
    (3, 10, 16, 10, 16, -1, False),  # 256 channels: four waves per cell
    (4, 9, 16, 12, 8, -1, False),    # 16 x 8: two waves, each with eight channels of x
    (5, 12, 4, 7, 16, 15, False),    # 4 x 16 in one wave, capped product
    (7, 6, 8, 11, 2, -1, False),     # 8 x 2: one tile, the y-gradient is added over the halves
    (3, 15, 16, 15, 16, 21, False),  # the largest rows the kernel takes, l from 0 to 21
    (2, 11, 4, 11, 4, 3, False),     # l1 + l2 = 22 capped at 3: four values of l
]
MFMA_SHAPES = {(8, 8), (4, 4), (8, 16), (16, 16), (16, 8), (4, 16), (8, 2)}


@pytest.mark.parametrize("mfma", [1, 0])
@pytest.mark.parametrize("B,l1,n1,l2,n2,maxl,diag", CASES)
def test_onepair_bwd(cabi, B, l1, n1, l2, n2, maxl, diag, mfma):
    """Both forms of the family: with the matrix-core kernel allowed (it takes the channel counts in MFMA_SHAPES) and
    without it."""
    if not mfma and ((n1, n2) != (8, 8) or diag):
        pytest.skip("the same kernel either way" if n1 * n2 <= 64 else "more than 64 channel slots: only the matrix-core kernel takes it")
    cabi.set_option("onepair_mfma", mfma)
    try:
        run_onepair(cabi, B, l1, n1, l2, n2, maxl, diag)
    finally:
        cabi.set_option("onepair_mfma", 1)


def run_onepair(cabi, B, l1, n1, l2, n2, maxl, diag):
    seed = 1300 + B
    xs = [U.seeded(seed, B, 2 * l1 + 1, n1)]
    ys = [U.seeded(seed + 1, B, 2 * l2 + 1, n2)]
    O = U.VecOracle(xs, ys, maxl, diag, gseed=seed + 100)
    gs = O.gs
    dxs, dys, dgs = [U.dev(a) for a in xs], [U.dev(a) for a in ys], [U.dev(a) for a in gs]
    dxg = [torch.full(a.shape, 3.0 - 2j, dtype=torch.complex64, device="cuda") for a in xs]
    dyg = [torch.full(a.shape, 3.0 - 2j, dtype=torch.complex64, device="cuda") for a in ys]
    cabi.so3vec_bwd(dxg, dyg, dgs, dxs, dys, accumulate=False, diag=diag)
    assert cabi.last_path() == ONEPAIR
    torch.cuda.synchronize()
    tag = "B%d (%d,%d)x(%d,%d) maxl %d diag %d" % (B, l1, n1, l2, n2, maxl, diag)
    O.check_bwd([U.host(dxg[0])], [U.host(dyg[0])], tag)
    dxg2, dyg2 = [a.clone() for a in dxg], [a.clone() for a in dyg]
    cabi.so3vec_bwd(dxg2, dyg2, dgs, dxs, dys, accumulate=True, diag=diag)
    assert cabi.last_path() == ONEPAIR
    torch.cuda.synchronize()
    O.check_bwd_onto([U.host(a) for a in dxg2], [U.host(a) for a in dyg2], [U.host(a) for a in dxg],
                     [U.host(a) for a in dyg], tag + " accumulated")


def test_onepair_leaves_the_rest_alone(cabi):
    # one gradient alone, two x parts, l1 + l2 above 21: other kernels
    x, y = [U.dev(U.seeded(1, 4, 21, 8))], [U.dev(U.seeded(2, 4, 21, 8))]
    want = ora.vec_fwd([U.host(x[0])], [U.host(y[0])])
    g = [U.dev(U.seeded(10 + i, *p.shape)) for i, p in enumerate(want)]
    xg = [torch.zeros_like(x[0])]
    cabi.so3vec_bwd(xg, None, g, x, y, accumulate=False)
    assert cabi.last_path() != ONEPAIR
    O = U.VecOracle([U.host(x[0])], [U.host(y[0])], -1, False, gs=[U.host(t) for t in g])
    O.check_bwd([U.host(xg[0])], None, "one gradient alone")
    x11, y11 = [U.dev(U.seeded(3, 2, 23, 3))], [U.dev(U.seeded(4, 2, 23, 4))]
    w11 = ora.vec_fwd([U.host(x11[0])], [U.host(y11[0])], 3)
    g11 = [U.dev(U.seeded(20 + i, *p.shape)) for i, p in enumerate(w11)]
    xg11, yg11 = [torch.zeros_like(x11[0])], [torch.zeros_like(y11[0])]
    cabi.so3vec_bwd(xg11, yg11, g11, x11, y11, accumulate=False)
    assert cabi.last_path() != ONEPAIR


# (the l1 = l2 = 15 case with 256 channels needs more LDS than the forward kernel asks for: other kernels take it)
FWD_CASES = [c for c in CASES if (c[2], c[4]) in MFMA_SHAPES and not c[6] and c[1] + c[3] >= 3 and c[0] != 33
             and (c[1], c[2]) != (15, 16)]


@pytest.mark.parametrize("B,l1,n1,l2,n2,maxl,diag", FWD_CASES)
def test_onepair_fwd_on_the_matrix_cores(cabi, B, l1, n1, l2, n2, maxl, diag):
    """The product itself for the channel counts of the matrix-core kernel: overwrite into garbage, accumulate on top, a block at a channel offset of a
    wider part (the other channels must stay as they were), and the same bits on a second run."""
    seed = 1700 + B
    xs = [U.seeded(seed, B, 2 * l1 + 1, n1)]
    ys = [U.seeded(seed + 1, B, 2 * l2 + 1, n2)]
    O = U.VecOracle(xs, ys, maxl, diag)
    dxs, dys = [U.dev(a) for a in xs], [U.dev(a) for a in ys]
    drs = [torch.full(p.shape, 7.0 + 1j, dtype=torch.complex64, device="cuda") for p in O.r32]
    cabi.so3vec_fwd(drs, dxs, dys, accumulate=False, diag=diag)
    assert cabi.last_path() == ONEPAIR
    torch.cuda.synchronize()
    tag = "fwd B%d (%d,%d)x(%d,%d) maxl %d" % (B, l1, n1, l2, n2, maxl)
    O.check_fwd([U.host(a) for a in drs], tag)
    start = [U.seeded(seed + 20 + k, *p.shape) for k, p in enumerate(O.r32)]
    drs2 = [U.dev(a) for a in start]
    cabi.so3vec_fwd(drs2, dxs, dys, accumulate=True, diag=diag)
    assert cabi.last_path() == ONEPAIR
    drs3 = [torch.empty_like(t) for t in drs]
    cabi.so3vec_fwd(drs3, dxs, dys, accumulate=False, diag=diag)
    torch.cuda.synchronize()
    O.check_fwd_onto([U.host(a) for a in drs2], start, tag + " onto")
    assert all(torch.equal(a.view(torch.float32), b.view(torch.float32)) for a, b in zip(drs, drs3))
    # part-level calls with a channel offset into wider parts
    l = min(l1 + l2, maxl if maxl >= 0 else l1 + l2)
    nn = n1 * n2
    wide = torch.full((B, 2 * l + 1, nn + 6), 5.0 - 3j, dtype=torch.complex64, device="cuda")
    cabi.so3part_cg_fwd(wide, dxs[0], dys[0], offs=4, accumulate=False)
    torch.cuda.synchronize()
    hw = U.host(wide)
    k = [p.shape[1] for p in O.r32].index(2 * l + 1)
    U.assert_parity(hw[:, :, 4:4 + nn], O.r32[k], O.r64[k], O.Sr[k], tag + " offset block")
    assert np.all(hw[:, :, :4] == np.complex64(5.0 - 3j)) and np.all(hw[:, :, 4 + nn:] == np.complex64(5.0 - 3j))


def test_vectors_of_several_parts_above_l7_go_pair_by_pair(cabi):
    """x parts l = 8, 9 and y parts l = 9, 10 with 4 channels each: forward and backward run one launch of the
    matrix-core single-pair kernels per (x part, y part) pair; product capped so that the oracle stays quick."""
    B, tau, maxl = 3, 4, 12
    xs = [U.seeded(40 + l, B, 2 * l + 1, tau) for l in (8, 9)]
    ys = [U.seeded(50 + l, B, 2 * l + 1, tau) for l in (9, 10)]
    O = U.VecOracle(xs, ys, maxl, False, gseed=77)
    dxs, dys, dgs = [U.dev(a) for a in xs], [U.dev(a) for a in ys], [U.dev(a) for a in O.gs]
    drs = [torch.full(p.shape, 7.0 + 1j, dtype=torch.complex64, device="cuda") for p in O.r32]
    cabi.so3vec_fwd(drs, dxs, dys, accumulate=False)
    assert cabi.last_path() == ONEPAIR
    torch.cuda.synchronize()
    O.check_fwd([U.host(a) for a in drs], "several parts above l = 7, forward")
    dxg = [torch.full(a.shape, 3.0 - 2j, dtype=torch.complex64, device="cuda") for a in xs]
    dyg = [torch.full(a.shape, 3.0 - 2j, dtype=torch.complex64, device="cuda") for a in ys]
    cabi.so3vec_bwd(dxg, dyg, dgs, dxs, dys, accumulate=False)
    assert cabi.last_path() == ONEPAIR
    torch.cuda.synchronize()
    O.check_bwd([U.host(a) for a in dxg], [U.host(a) for a in dyg], "several parts above l = 7, backward")
