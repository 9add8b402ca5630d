"""GPU parity of the six part-level entry points, called through the C ABI, against the CPU oracle on the same
seeded inputs.  Every real component must pass the parity rules of tests/gpu_util.py (the gate
|gpu - cpu| <= 1e-6 + 1e-5 |cpu|, or one of the two stated rules for elements whose float32 sum nearly cancels)."""
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
    return c


SHAPES = [
    # (B, l1, l2, l, n1, n2)
    (1024, 1, 1, 1, 16, 16),     # configuration 1 of the benchmark list
    (3, 0, 0, 0, 1, 1),
    (2, 1, 1, 2, 1, 1),
    (5, 2, 3, 4, 4, 8),
    (7, 2, 3, 1, 3, 5),          # odd channel counts
    (4, 4, 4, 4, 16, 16),
    (3, 4, 3, 7, 8, 2),
    (2, 3, 3, 0, 32, 32),
    (2, 6, 5, 3, 4, 4),
    (2, 10, 10, 7, 8, 8),        # large l: shape-agnostic kernels
    (1, 2, 2, 2, 70, 3),         # n1*n2 not a multiple of the wave
    (300, 1, 2, 3, 2, 2),
    (3, 4, 4, 8, 4, 4),          # the largest and the smallest l of the (4, 4) pair
    (3, 4, 4, 0, 8, 8),
    (9, 0, 3, 3, 16, 4),
    (2, 6, 6, 6, 2, 4),          # operands above l = 4, product l up to 6
    (2, 5, 6, 1, 8, 2),
    (2, 6, 6, 12, 2, 2),         # operands of l = 6 into l = 12: beyond the l range of the unrolled kernels' pair records
    (3, 6, 5, 9, 4, 2),
    (5, 2, 3, 4, 32, 32),        # configuration 2's triple: the single-triple backward kernel, 32 channels of y
    (3, 3, 2, 1, 16, 64),        # ... 64
    (3, 4, 4, 8, 64, 16),        # ... 16
    (2, 0, 4, 4, 16, 32),
    (2, 4, 0, 4, 128, 32),
    (6, 1, 1, 0, 32, 16),
]


def run_part(cabi, B, l1, l2, l, n1, n2, diag, seed, force_generic):
    cabi.set_option("force_generic", int(force_generic))
    if diag:
        n2 = n1
    x = U.seeded(seed, B, 2 * l1 + 1, n1)
    y = U.seeded(seed + 1, B, 2 * l2 + 1, n2)
    nout = n1 if diag else n1 * n2
    offs = 3
    r0 = U.seeded(seed + 2, B, 2 * l + 1, nout + 5)
    g = U.seeded(seed + 3, B, 2 * l + 1, nout + 5)
    xg0 = U.seeded(seed + 4, *x.shape)
    yg0 = U.seeded(seed + 5, *y.shape)
    ops = (ora.DIAG_FWD, ora.DIAG_BACK0, ora.DIAG_BACK1) if diag else (ora.CG_FWD, ora.CG_BACK0, ora.CG_BACK1)
    fns = ((cabi.so3part_diagcg_fwd, cabi.so3part_diagcg_back0, cabi.so3part_diagcg_back1) if diag else
           (cabi.so3part_cg_fwd, cabi.so3part_cg_back0, cabi.so3part_cg_back1))

    def both(prec, zero_start):
        c = (lambda a: a.astype(np.complex128)) if prec == 64 else (lambda a: a.copy())
        z = (lambda a: np.zeros_like(c(a))) if zero_start else c
        r, xg, yg = z(r0), z(xg0), z(yg0)
        ora.part_op(ops[0], r, c(x), c(y), offs)
        ora.part_op(ops[1], c(g), xg, c(y), offs)
        ora.part_op(ops[2], c(g), c(x), yg, offs)
        return r, xg, yg

    # sums of the moduli of each element's terms (rule C of the parity check)
    Sr = ora.part_term_sums(ops[0], r0, x, y, offs)
    Sxg = ora.part_term_sums(ops[1], g, x, y, offs)
    Syg = ora.part_term_sums(ops[2], g, x, y, offs)

    dx, dy, dg = U.dev(x), U.dev(y), U.dev(g)
    # accumulate (reference semantics): the existing value is one more term of every sum
    r32, xg32, yg32 = both(32, False)
    r64, xg64, yg64 = both(64, False)
    dr, dxg, dyg = U.dev(r0), U.dev(xg0), U.dev(yg0)
    fns[0](dr, dx, dy, offs, True)
    fns[1](dxg, dg, dy, offs, True)
    fns[2](dyg, dg, dx, offs, True)
    torch.cuda.synchronize()
    tag = "B%d (%d,%d,%d) n%dx%d diag=%d" % (B, l1, l2, l, n1, n2, diag)
    U.assert_parity(U.host(dr), r32, r64, Sr + np.abs(r0), "fwd " + tag)
    U.assert_parity(U.host(dxg), xg32, xg64, Sxg + np.abs(xg0), "back0 " + tag)
    U.assert_parity(U.host(dyg), yg32, yg64, Syg + np.abs(yg0), "back1 " + tag)
    # channels outside the block stay untouched
    assert np.array_equal(U.host(dr)[:, :, :offs], r0[:, :, :offs])
    assert np.array_equal(U.host(dr)[:, :, offs + nout:], r0[:, :, offs + nout:])
    # overwrite mode writes exactly the block / the gradient: the oracle started from zeros
    r32, xg32, yg32 = both(32, True)
    r64, xg64, yg64 = both(64, True)
    dr, dxg, dyg = U.dev(r0), U.dev(xg0), U.dev(yg0)
    fns[0](dr, dx, dy, offs, False)
    fns[1](dxg, dg, dy, offs, False)
    fns[2](dyg, dg, dx, offs, False)
    torch.cuda.synchronize()
    blk = slice(offs, offs + nout)
    U.assert_parity(U.host(dr)[:, :, blk], r32[:, :, blk], r64[:, :, blk], Sr[:, :, blk], "fwd overwrite " + tag)
    assert np.array_equal(U.host(dr)[:, :, :offs], r0[:, :, :offs])
    assert np.array_equal(U.host(dr)[:, :, offs + nout:], r0[:, :, offs + nout:])
    U.assert_parity(U.host(dxg), xg32, xg64, Sxg, "back0 overwrite " + tag)
    U.assert_parity(U.host(dyg), yg32, yg64, Syg, "back1 overwrite " + tag)
    return cabi.last_path()


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("diag", [False, True])
def test_part_generic(cabi, shape, diag):
    assert run_part(cabi, *shape, diag, seed=100, force_generic=True) == 1


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("diag", [False, True])
def test_part_default_path(cabi, shape, diag):
    run_part(cabi, *shape, diag, seed=200, force_generic=False)


def test_batch_broadcast(cabi):
    # x with batch 1 (core/Gpart.hpp:168-185): forward broadcasts, back0 sums over the batch
    cabi.set_option("force_generic", 0)
    B, l1, l2, l, n = 6, 2, 2, 2, 4
    x = U.seeded(1, 1, 2 * l1 + 1, n)
    y = U.seeded(2, B, 2 * l2 + 1, n)
    r32 = ora.cg_fwd(x, y, l)
    g = U.seeded(3, *r32.shape)
    xg32, yg32 = ora.cg_bwd(g, x, y)
    xg64, yg64 = ora.cg_bwd(g.astype(np.complex128), x.astype(np.complex128), y.astype(np.complex128))
    Sxg = ora.part_term_sums(ora.CG_BACK0, g, x, y)
    Syg = ora.part_term_sums(ora.CG_BACK1, g, x, y)
    dx, dy, dg = U.dev(x), U.dev(y), U.dev(g)
    dr = torch.zeros(B, 2 * l + 1, n * n, dtype=torch.complex64, device="cuda")
    cabi.so3part_cg_fwd(dr, dx, dy)
    dxg, dyg = torch.zeros_like(dx), torch.zeros_like(dy)
    cabi.so3part_cg_back0(dxg, dg, dy)
    cabi.so3part_cg_back1(dyg, dg, dx)
    torch.cuda.synchronize()
    assert U.gate_excess(U.host(dr), r32) <= 1.0
    U.assert_parity(U.host(dxg), xg32, xg64, Sxg, "bcast back0")
    U.assert_parity(U.host(dyg), yg32, yg64, Syg, "bcast back1")


def test_strided_views(cabi):
    # permuted / sliced tensors (python/tests/bug1.py): arbitrary strides must give the same numbers
    cabi.set_option("force_generic", 0)
    B, l1, l2, l, n1, n2 = 5, 1, 2, 2, 3, 4
    x = U.seeded(11, B, 2 * l1 + 1, n1)
    y = U.seeded(12, B, 2 * l2 + 1, n2)
    want = ora.cg_fwd(x, y, l)
    dx = U.dev(np.ascontiguousarray(x.transpose(2, 0, 1))).permute(1, 2, 0)           # channel-major storage
    dy = U.dev(np.repeat(y, 2, axis=2))[:, :, ::2]                                     # channel stride 2
    big = torch.zeros(B, 2 * l + 1, 2 * n1 * n2, dtype=torch.complex64, device="cuda")
    dr = big[:, :, n1 * n2 // 2: n1 * n2 // 2 + n1 * n2]                                # offset view, row stride > n
    cabi.so3part_cg_fwd(dr, dx, dy)
    torch.cuda.synchronize()
    assert U.gate_excess(U.host(dr), want) <= 1.0
    assert float(big[:, :, :n1 * n2 // 2].abs().max()) == 0.0


def test_grid_cells(cabi):
    # 5-D (b, g0, g1, m, n) with a grid-less second operand (core/Gpart.hpp:416-432)
    cabi.set_option("force_generic", 0)
    B, G0, G1, l1, l2, l, n = 2, 2, 3, 1, 1, 2, 2
    x = U.seeded(21, B * G0 * G1, 3, n)
    y = U.seeded(22, B, 3, n)
    yfull = np.repeat(y, G0 * G1, axis=0)
    want = ora.cg_fwd(x, yfull, l).reshape(B, G0, G1, 2 * l + 1, n * n)
    dx = U.dev(x).reshape(B, G0, G1, 3, n)
    dy = U.dev(y)
    dr = torch.zeros(B, G0, G1, 2 * l + 1, n * n, dtype=torch.complex64, device="cuda")
    cabi.so3part_cg_fwd(dr, dx, dy)
    torch.cuda.synchronize()
    assert U.gate_excess(U.host(dr), want) <= 1.0


def test_empty_batch(cabi):
    z = torch.zeros(0, 3, 4, dtype=torch.complex64, device="cuda")
    r = torch.zeros(0, 3, 16, dtype=torch.complex64, device="cuda")
    cabi.so3part_cg_fwd(r, z, z)
    cabi.so3part_cg_back0(z, r, z)
    torch.cuda.synchronize()


def test_host_tensor_rejected(cabi):
    x = torch.zeros(2, 3, 4, dtype=torch.complex64)
    r = torch.zeros(2, 3, 16, dtype=torch.complex64)
    with pytest.raises(cabi.GelibHipError) as e:
        cabi.so3part_cg_fwd(r, x, x)
    assert e.value.status == 8
