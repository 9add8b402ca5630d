"""GPU parity of the SO3vec-level entry points (all triples in one call) against the CPU oracle."""
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


CASES = [
    # (B, tau_x, tau_y, maxl)
    (33, {l: 16 for l in range(5)}, {l: 16 for l in range(5)}, 4),      # headline type, small batch
    (9, {l: 16 for l in range(5)}, {l: 16 for l in range(5)}, -1),
    (4, {0: 2, 1: 3, 2: 2}, {1: 2, 2: 1}, -1),
    (4, {0: 1, 2: 4}, {0: 4, 1: 4, 3: 2}, 3),
    (3, {l: 4 for l in range(3)}, {l: 4 for l in range(3)}, 2),
    (2, {10: 8}, {10: 8}, -1),                                           # configuration 5 type
    (5, {l: 8 for l in range(7)}, {l: 8 for l in range(7)}, 6),
    (6, {0: 2, 3: 4, 5: 8, 6: 2}, {1: 4, 4: 2, 6: 8}, 6),                # operands up to l = 6, mixed channel counts
    (3, {5: 16}, {6: 4}, 5),                                             # one pair with l1, l2 above 4, capped
    (2, {1: 4}, {1: 128}, -1),                                           # more channels of y than a wave has lanes
    (2, {0: 2, 1: 3}, {1: 128, 2: 96}, 2),                               # ... and counts that are not powers of two
]


def run_vec(cabi, B, tx, ty, maxl, diag, seed, force_generic):
    cabi.set_option("force_generic", int(force_generic))
    if diag:
        ty = {l: tx[min(tx)] for l in ty}
        tx = {l: tx[min(tx)] for l in tx}
    xs = [U.seeded(seed + l, B, 2 * l + 1, n) for l, n in sorted(tx.items())]
    ys = [U.seeded(seed + 50 + l, B, 2 * l + 1, n) for l, n in sorted(ty.items())]
    O = U.VecOracle(xs, ys, maxl, diag, gseed=seed + 100)
    r32, gs = O.r32, O.gs
    dxs, dys, dgs = [U.dev(a) for a in xs], [U.dev(a) for a in ys], [U.dev(a) for a in gs]
    # overwrite mode into garbage: every channel of every part must be written exactly once
    drs = [torch.full(p.shape, 7.0 + 1j, dtype=torch.complex64, device="cuda") for p in r32]
    cabi.so3vec_fwd(drs, dxs, dys, accumulate=False, diag=diag)
    path_fwd = cabi.last_path()
    dxg = [torch.full(a.shape, 3.0 - 2j, dtype=torch.complex64, device="cuda") for a in xs]
    dyg = [torch.full(a.shape, 3.0 - 2j, dtype=torch.complex64, device="cuda") for a in ys]
    cabi.so3vec_bwd(dxg, dyg, dgs, dxs, dys, accumulate=False, diag=diag)
    path_bwd = cabi.last_path()
    torch.cuda.synchronize()
    tag = "B%d %s x %s maxl %d diag %d" % (B, tx, ty, maxl, diag)
    O.check_fwd([U.host(a) for a in drs], tag)
    O.check_bwd([U.host(a) for a in dxg], [U.host(a) for a in dyg], tag)
    # accumulate mode adds on top; back0-only and back1-only calls
    drs2 = [a.clone() for a in drs]
    cabi.so3vec_fwd(drs2, dxs, dys, accumulate=True, diag=diag)
    dxg2 = [torch.zeros_like(a) for a in dxs]
    dyg2 = [torch.zeros_like(a) for a in dys]
    cabi.so3vec_bwd(dxg2, None, dgs, dxs, dys, accumulate=True, diag=diag)
    cabi.so3vec_bwd(None, dyg2, dgs, dxs, dys, accumulate=True, diag=diag)
    torch.cuda.synchronize()
    for a, b in zip(drs2, drs):   # the product added onto itself: an exact doubling, up to the rounding of the add
        assert U.gate_excess(U.host(a), 2 * U.host(b)) <= 1.0
    # one gradient per call, added onto zeros: held to the same rules as the fused call
    O.check_bwd([U.host(a) for a in dxg2], [U.host(a) for a in dyg2], tag + " (one gradient per call)")
    return path_fwd, path_bwd


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("diag", [False, True])
def test_vec_generic(cabi, case, diag):
    assert run_vec(cabi, *case, diag, seed=300, force_generic=True) == (1, 1)


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("diag", [False, True])
def test_vec_default_path(cabi, case, diag):
    run_vec(cabi, *case, diag, seed=400, force_generic=False)


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("diag", [False, True])
def test_vec_without_pair_split(cabi, case, diag):
    """Launches with few cells (every case here) deal the pairs of a cell to several blocks of the unrolled backward
    kernels and add their partial sums in a second kernel; with that switched off one block takes all pairs of its
    cells, as in launches with many cells.  Both ways to the same parity rules; the fixed order of additions makes
    each of them reproducible bit for bit."""
    cabi.set_option("unrolled_bwd_split", 0)
    try:
        run_vec(cabi, *case, diag, seed=400, force_generic=False)
    finally:
        cabi.set_option("unrolled_bwd_split", 1)


def test_pair_split_is_reproducible_and_respects_accumulate(cabi):
    cabi.set_option("force_generic", 0)
    B, tau = 40, {l: 16 for l in range(5)}
    xs = [U.seeded(1 + l, B, 2 * l + 1, n) for l, n in tau.items()]
    ys = [U.seeded(11 + l, B, 2 * l + 1, n) for l, n in tau.items()]
    O = U.VecOracle(xs, ys, 4, False, gseed=21)
    dxs, dys, dgs = [U.dev(a) for a in xs], [U.dev(a) for a in ys], [U.dev(a) for a in O.gs]
    outs = []
    for smax in (16, 16, 3):
        cabi.set_option("unrolled_bwd_split_max", smax)
        dxg = [torch.full(a.shape, 3.0 - 2j, dtype=torch.complex64, device="cuda") for a in xs]
        dyg = [torch.full(a.shape, 3.0 - 2j, dtype=torch.complex64, device="cuda") for a in ys]
        cabi.so3vec_bwd(dxg, dyg, dgs, dxs, dys, accumulate=False)
        assert cabi.last_path() == 2
        torch.cuda.synchronize()
        outs.append([U.host(a) for a in dxg + dyg])
        O.check_bwd(outs[-1][:5], outs[-1][5:], "pair split, at most %d blocks per cell" % smax)
    cabi.set_option("unrolled_bwd_split_max", 16)
    assert all(np.array_equal(a, b) for a, b in zip(outs[0], outs[1]))
    sx = [U.seeded(31 + i, *a.shape) for i, a in enumerate(xs)]
    sy = [U.seeded(41 + i, *a.shape) for i, a in enumerate(ys)]
    dxg, dyg = [U.dev(a) for a in sx], [U.dev(a) for a in sy]
    cabi.so3vec_bwd(dxg, dyg, dgs, dxs, dys, accumulate=True)
    torch.cuda.synchronize()
    O.check_bwd_onto([U.host(a) for a in dxg], [U.host(a) for a in dyg], sx, sy, "pair split, accumulate")


@pytest.mark.parametrize("case", [
    (3, {l: 8 for l in range(7)}, {l: 8 for l in range(7)}, -1),       # L = 6 uncapped: product l up to 12
    (4, {2: 4, 5: 8, 6: 2}, {3: 4, 6: 4}, 9),                          # parts missing, capped between 6 and 12
    (2, {6: 16}, {6: 4}, -1),                                          # one pair, l = 0..12
    (5, {0: 2, 5: 2}, {1: 4, 6: 1}, 11),
    (3, {l: 6 for l in range(7)}, {l: 6 for l in range(7)}, -1),       # channel counts that are not powers of two
    (4, {2: 6, 5: 2}, {1: 12, 6: 5}, 9),
])
def test_operands_above_l4_product_above_l6(cabi, case):
    """CGproduct of operands up to l = 6 that reaches above l = 6: the triples up to l = 6 on the unrolled kernels built
    for them, the rest forward on the any-l kernels and backward on the unrolled instantiation for l = 7..12, which adds
    onto the first launch's gradients; g is read once."""
    assert run_vec(cabi, *case, False, seed=520, force_generic=False) == (2, 2)
    cabi.set_option("unrolled_bwd_l6_split", 0)
    try:
        assert run_vec(cabi, *case, False, seed=520, force_generic=False)[1] != 2     # the striped any-l kernels
    finally:
        cabi.set_option("unrolled_bwd_l6_split", 1)


def test_absent_output_part_keeps_offsets(cabi):
    # a product part that is missing is skipped; the blocks of the other parts stay where they are
    cabi.set_option("force_generic", 0)
    tx = {0: 2, 1: 2}
    xs = [U.seeded(1 + l, 3, 2 * l + 1, n) for l, n in tx.items()]
    ys = [U.seeded(9 + l, 3, 2 * l + 1, n) for l, n in tx.items()]
    full = ora.vec_fwd(xs, ys)                      # parts l = 0, 1, 2
    drs = [torch.zeros(p.shape, dtype=torch.complex64, device="cuda") for p in (full[0], full[2])]
    cabi.so3vec_fwd(drs, [U.dev(a) for a in xs], [U.dev(a) for a in ys], accumulate=True)
    torch.cuda.synchronize()
    assert U.gate_excess(U.host(drs[0]), full[0]) <= 1.0
    assert U.gate_excess(U.host(drs[1]), full[2]) <= 1.0


def test_parts_in_any_order(cabi):
    cabi.set_option("force_generic", 0)
    xs = [U.seeded(1 + l, 2, 2 * l + 1, 2) for l in range(3)]
    ys = [U.seeded(7 + l, 2, 2 * l + 1, 2) for l in range(3)]
    want = ora.vec_fwd(xs, ys, 2)
    drs = [torch.zeros(p.shape, dtype=torch.complex64, device="cuda") for p in want]
    cabi.so3vec_fwd(drs[::-1], [U.dev(a) for a in xs[::-1]], [U.dev(a) for a in ys], accumulate=False)
    torch.cuda.synchronize()
    for a, b in zip(drs, want):
        assert U.gate_excess(U.host(a), b) <= 1.0


@pytest.mark.parametrize("case", [
    (6, {0: 3, 1: 5, 2: 12}, {1: 6, 2: 7, 4: 3}, -1),      # nothing is a power of two; product l up to 6
    (33, {l: 12 for l in range(5)}, {l: 12 for l in range(5)}, 4),
    (70, {1: 1, 3: 3}, {2: 5}, 4),                           # 5 and 15 lane slots per cell: many cells per run
    (3, {2: 24}, {3: 40}, -1),                               # 24 x 40 channels: several runs per cell, n2 padded to 64
    # the first operand's channels are not rounded up where a cell's lane slots still fill whole runs of 64
    (5, {0: 3, 2: 3}, {1: 64, 2: 32}, -1),                   # 3 x 64 slots: three runs; 3 x 32: rounded up to 4 x 32
    (4, {1: 20, 3: 12}, {0: 24, 2: 16}, 4),                  # 20 x 32, 12 x 32, 20 x 16, 12 x 16 slots
    (2, {0: 192, 1: 192}, {0: 192, 1: 192}, -1),             # Diag: 192 channels, three runs per cell (CGproduct: 192 x 256)
])
@pytest.mark.parametrize("diag", [False, True])
def test_channel_counts_that_are_not_powers_of_two(cabi, case, diag):
    """The unrolled backward kernels round the channel counts up to powers of two for their lane layout; lanes
    beyond the real channels idle.  Both gradients still come from the fused kernels (path 2).  The lane-per-channel
    Diag kernels, which would take the Diag cases first, are switched off here; tests/test_gpu_diag6.py covers them."""
    cabi.set_option("diag6", 0)
    try:
        assert run_vec(cabi, *case, diag, seed=500, force_generic=False) == (2, 2)
    finally:
        cabi.set_option("diag6", 1)


def test_channel_counts_that_are_not_powers_of_two_above_l4(cabi):
    """CGproduct of operands up to l = 6, capped at l = 6: forward on the unrolled kernel built for them (even channel
    counts of the first operand), backward on its instantiation with padded lane slots."""
    assert run_vec(cabi, 4, {2: 6, 5: 2}, {1: 12, 6: 5}, 6, False, seed=510, force_generic=False) == (2, 2)
    assert run_vec(cabi, 3, {l: 6 for l in range(7)}, {l: 6 for l in range(7)}, 6, False, seed=511,
                   force_generic=False) == (2, 2)


@pytest.mark.parametrize("case", [
    (3, {l: 1 for l in range(17)}, {0: 2}, -1),      # 17 operand parts: more than the fused kernels' part lists hold
    (2, {32: 1}, {32: 1}, -1),                        # 65 product parts, l = 0..64
])
def test_more_parts_than_the_fused_kernels_take(cabi, case):
    """The reference's loop over triples has no limit on the number of parts (core/Gvec.hpp:311-345); vectors beyond the
    fused kernels' argument lists run one launch per triple on the shape-agnostic kernels going forward, and one launch
    per pair of parts on the single-pair kernels (or again per triple) going backward."""
    fwd, bwd = run_vec(cabi, *case, False, seed=800, force_generic=False)
    assert fwd == 1 and bwd in (1, 5)


def test_tuning_options_leave_the_results_alone(cabi):
    """The launch-shape options (cells per tile and bytes per block of the forward pass, LDS per block of the backward
    pass) and the switches between kernels that compute the same sums (the Diag backward kernel with fixed sets of l2,
    the single-triple kernel, the paired row numbers of the matrix-core kernel) change timings only.  Options that keep
    the order of every sum are held to the same bits, the others to the parity rules."""
    cabi.set_option("force_generic", 0)

    def product(tx, ty, maxl, diag, seed, B=37):
        xs = [U.dev(U.seeded(seed + l, B, 2 * l + 1, n)) for l, n in sorted(tx.items())]
        ys = [U.dev(U.seeded(seed + 40 + l, B, 2 * l + 1, n)) for l, n in sorted(ty.items())]
        tau = cabi.so3type_product(tx, ty, maxl, diag)
        rs = [torch.empty(B, 2 * l + 1, n, dtype=torch.complex64, device="cuda") for l, n in sorted(tau.items())]
        cabi.so3vec_fwd(rs, xs, ys, accumulate=False, diag=diag)
        xg, yg = [torch.empty_like(t) for t in xs], [torch.empty_like(t) for t in ys]
        cabi.so3vec_bwd(xg, yg, rs, xs, ys, accumulate=False, diag=diag)
        torch.cuda.synchronize()
        return [U.host(t) for t in rs], [U.host(t) for t in xg + yg]

    def same_bits(a, b):
        return all(np.array_equal(p.view(np.float32), q.view(np.float32)) for p, q in zip(a, b))

    def close(a, b):   # two float32 evaluations of the same sums in different orders
        return all(np.max(np.abs(p - q)) <= 2e-5 * max(1.0, np.max(np.abs(p))) for p, q in zip(a, b))

    L4 = {l: 4 for l in range(5)}
    L6 = {l: 64 for l in range(7)}
    cases = [
        # option, default, other values, workload, forward bits kept, backward bits kept
        ("fwd_cell_tile", -1, (0, 16, 4096), (L4, L4, 4, False), True, True),
        ("fwd_block_bytes", 0, (32768, 262144), (L4, L4, -1, False), True, True),
        ("bwd_lds_target", 40960, (16384, 65536), (L4, L4, 4, False), True, False),
        ("diag6_sets", 1, (0,), (L6, L6, 6, True), True, True),
        ("unrolled_bwd_one", 1, (0,), ({2: 8}, {3: 8}, 1, False), True, False),     # capped at l = 1: one triple
        ("onepair_mfma_paired", 1, (0,), ({7: 8}, {7: 8}, -1, False), True, False),
    ]
    for name, default, others, (tx, ty, maxl, diag), fwd_bits, bwd_bits in cases:
        r0, g0 = product(tx, ty, maxl, diag, seed=900)
        try:
            for v in others:
                cabi.set_option(name, v)
                r1, g1 = product(tx, ty, maxl, diag, seed=900)
                assert same_bits(r0, r1) if fwd_bits else close(r0, r1), (name, v)
                assert same_bits(g0, g1) if bwd_bits else close(g0, g1), (name, v)
        finally:
            cabi.set_option(name, default)
