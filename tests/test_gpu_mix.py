"""Channel mixing (the linear layer that consumes a product) through the C-ABI, against numpy's complex128 matmul.

Tolerance: the matrix cores add the 2 n_in real terms of an output one after the other in float32, so the error of an
output is a rounding error of its sum and is measured against the size of that sum, not of its (possibly cancelling)
value:  |gpu - exact| <= 1e-6 + 4 eps32 * sum_c |x_c| |V_co|.  A dropped term, a wrong sign or a transposed weight
is off by the size of a term, 10^5 times more."""
import numpy as np
import pytest

from tests import gpu_util as U

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def cabi():
    assert torch.cuda.is_available()
    from gelib_amd import cabi as c
    c.lib()
    return c


def rand(shape, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return torch.view_as_complex(torch.randn(*shape, 2, device="cuda", generator=g))


# (leading extents, n_in, n_out): single and several tiles of output, reductions shorter and longer than one step of
# 16 channels, row counts that are not multiples of the 64 rows of a wave, and the wide-output (gradient) shapes
CASES = [
    ((64,), 16, 16), ((1,), 2, 1), ((7, 3), 6, 5), ((100, 5), 256, 16), ((33, 9), 48, 16), ((130,), 34, 3),
    ((40, 3), 64, 32), ((40, 3), 20, 24), ((17, 5), 40, 64), ((9, 7), 96, 40), ((65,), 16, 256), ((31, 3), 32, 300),
    ((12, 9), 8, 70), ((257,), 1280, 16),
    # rows of 2 KB and more run on the LDS-staged kernel: a last step that is partly outside the row, two and eight
    # tiles of output, fewer rows than the 32 of a wave
    ((70,), 258, 5), ((33, 3), 300, 24), ((20, 3), 260, 70), ((5,), 1024, 16), ((3, 7), 514, 128),
    # many tiles of output: an odd number of output channels keeps the stores narrow, an even one sends them through LDS
    ((50,), 8, 35), ((333,), 16, 130), ((260,), 16, 64), ((129, 3), 14, 1000), ((64,), 16, 34),
]


@pytest.mark.parametrize("lead,n_in,n_out", CASES)
@pytest.mark.parametrize("adjoint", [False, True])
def test_mix_channels(cabi, lead, n_in, n_out, adjoint):
    x = rand(lead + (n_in,), 1)
    w = rand((n_out, n_in) if adjoint else (n_in, n_out), 2)
    r = torch.full(lead + (n_out,), float("nan"), dtype=torch.complex64, device="cuda")
    cabi.part_mix_channels(r, x, w, adjoint=adjoint)
    hx, hw = U.host(x).astype(np.complex128), U.host(w).astype(np.complex128)
    v = hw.conj().T if adjoint else hw
    want = hx @ v
    tol = 1e-6 + 4 * np.finfo(np.float32).eps * (np.abs(hx) @ np.abs(v))
    got = U.host(r)
    assert np.isfinite(got.view(np.float32)).all()
    err = np.abs(got - want)
    assert (err <= tol).all(), "mix %s %d %d %s: worst error / tolerance %.2f" % (lead, n_in, n_out, adjoint, (err / tol).max())


WGRAD_CASES = [
    ((64,), 16, 16), ((1,), 2, 1), ((7, 3), 6, 5), ((1000, 5), 256, 16), ((33, 9), 48, 16), ((130,), 34, 3),
    ((400, 3), 64, 32), ((40, 3), 20, 24), ((170, 5), 40, 64), ((9, 7), 96, 40), ((650,), 16, 256), ((31, 3), 32, 70),
    ((5000,), 130, 16), ((2, 2049), 8, 8),
]


@pytest.mark.parametrize("lead,n_in,n_out", WGRAD_CASES)
def test_mix_channels_wgrad(cabi, lead, n_in, n_out):
    """wg = sum over the rows of conj(x)^T g.  Tolerance as above, against the size of the sum: the partial sums of the
    row ranges are float32 and are added in float32."""
    x = rand(lead + (n_in,), 5)
    g = rand(lead + (n_out,), 6)
    wg = torch.full((n_in, n_out), float("nan"), dtype=torch.complex64, device="cuda")
    cabi.part_mix_channels_wgrad(wg, x, g)
    hx = U.host(x).astype(np.complex128).reshape(-1, n_in)
    hg = U.host(g).astype(np.complex128).reshape(-1, n_out)
    want = hx.conj().T @ hg
    tol = 1e-6 + 4 * np.finfo(np.float32).eps * (np.abs(hx).T @ np.abs(hg))
    got = U.host(wg)
    assert np.isfinite(got.view(np.float32)).all()
    err = np.abs(got - want)
    assert (err <= tol).all(), "wgrad %s %d %d: worst error / tolerance %.2f" % (lead, n_in, n_out, (err / tol).max())
    wg2 = torch.empty_like(wg)
    cabi.part_mix_channels_wgrad(wg2, x, g)
    assert torch.equal(torch.view_as_real(wg), torch.view_as_real(wg2))     # fixed summation order


def test_mix_channels_long_rows_on_the_short_step_kernel(cabi):
    x = rand((67, 3, 384), 3)
    w = rand((384, 16), 4)
    r0 = torch.empty(67, 3, 16, dtype=torch.complex64, device="cuda")
    r1 = torch.empty_like(r0)
    cabi.part_mix_channels(r0, x, w)
    cabi.set_option("mix_long", 0)
    try:
        cabi.part_mix_channels(r1, x, w)
    finally:
        cabi.set_option("mix_long", 1)
    want = U.host(x).astype(np.complex128) @ U.host(w).astype(np.complex128)
    tol = 1e-6 + 4 * np.finfo(np.float32).eps * (np.abs(U.host(x)).astype(np.float64) @ np.abs(U.host(w)).astype(np.float64))
    for r in (r0, r1):
        assert (np.abs(U.host(r) - want) <= tol).all()


def test_mix_channels_wide_and_narrow_stores_agree(cabi):
    x = rand((77, 5, 16), 7)
    w = rand((200, 16), 8)
    r0 = torch.empty(77, 5, 200, dtype=torch.complex64, device="cuda")
    r1 = torch.empty_like(r0)
    r2 = torch.empty_like(r0)
    cabi.part_mix_channels(r0, x, w, adjoint=True)      # the kernel that walks along the output
    cabi.set_option("mix_wide", 0)
    try:
        cabi.part_mix_channels(r2, x, w, adjoint=True)  # one wave per four tiles, stores through LDS
        cabi.set_option("mix_wide_store", 0)
        cabi.part_mix_channels(r1, x, w, adjoint=True)  # stores straight from the registers
    finally:
        cabi.set_option("mix_wide_store", 1)
        cabi.set_option("mix_wide", 1)
    assert torch.equal(torch.view_as_real(r0), torch.view_as_real(r1))
    assert torch.equal(torch.view_as_real(r2), torch.view_as_real(r1))


def test_mix_channels_rejects(cabi):
    x = rand((8, 3), 1)
    w = rand((3, 4), 2)
    r = torch.empty(8, 4, dtype=torch.complex64, device="cuda")
    with pytest.raises(cabi.GelibHipError):
        cabi.part_mix_channels(r, x, w)     # an odd number of input channels
    assert not cabi.mix_channels_ok(x)


def test_mix_channels_random_shapes(cabi):
    """Random draws over all three operations and all kernels: row counts around the 32 and 64 rows of a wave, channel
    counts around the tile sizes (16, 32, 64, 128 floats), long and short rows."""
    rng = np.random.default_rng(2024)
    eps = np.finfo(np.float32).eps
    pick = lambda: int(rng.choice([2, 4, 6, 8, 14, 16, 18, 30, 32, 34, 62, 64, 66, 126, 128, 130, 254, 256, 258, 300, 514]))
    for draw in range(150):
        rows = int(rng.choice([1, 2, 31, 32, 33, 63, 64, 65, 100, 257, 1000]))
        n_in = pick()
        n_out = int(rng.choice([1, 3, 5, 8, 15, 16, 17, 24, 31, 32, 33, 48, 64, 65, 100, 130, 256, 400]))
        what = draw % 3
        x = rand((rows, n_in), 100 + draw)
        hx = U.host(x).astype(np.complex128)
        tag = "draw %d: rows %d n_in %d n_out %d op %d" % (draw, rows, n_in, n_out, what)
        if what == 2:
            g = rand((rows, n_out), 500 + draw)
            wg = torch.full((n_in, n_out), float("nan"), dtype=torch.complex64, device="cuda")
            cabi.part_mix_channels_wgrad(wg, x, g)
            hg = U.host(g).astype(np.complex128)
            want, scale, got = hx.conj().T @ hg, np.abs(hx).T @ np.abs(hg), U.host(wg)
        else:
            w = rand((n_out, n_in) if what else (n_in, n_out), 500 + draw)
            r = torch.full((rows, n_out), float("nan"), dtype=torch.complex64, device="cuda")
            cabi.part_mix_channels(r, x, w, adjoint=bool(what))
            v = U.host(w).astype(np.complex128)
            v = v.conj().T if what else v
            want, scale, got = hx @ v, np.abs(hx) @ np.abs(v), U.host(r)
        assert np.isfinite(got.view(np.float32)).all(), tag
        assert (np.abs(got - want) <= 1e-6 + 4 * eps * scale).all(), tag


def test_mix_channels_row_strides(cabi):
    """The C entry points take row strides: a block of channels of a wider tensor in, a block of a wider tensor out."""
    rows, n_in, n_out = 300, 40, 16
    xw = rand((rows, 64), 11)                 # x = channels 8..47 of a 64-channel tensor
    rw = torch.zeros(rows, 24, dtype=torch.complex64, device="cuda")   # r = channels 4..19 of a 24-channel tensor
    w = rand((n_in, n_out), 12)
    x, r = xw[:, 8:8 + n_in], rw[:, 4:4 + n_out]
    L = cabi.lib()
    ws, nbytes = cabi.mix_workspace(0, rows, n_in, n_out, "cuda")
    cabi.check(L.gelib_hip_part_mix_channels(r.data_ptr(), x.data_ptr(), w.data_ptr(), rows, n_in, n_out, 24, 64, 0,
                                             ws.data_ptr(), nbytes, None))
    want = U.host(x.contiguous()).astype(np.complex128) @ U.host(w).astype(np.complex128)
    tol = 1e-6 + 4 * np.finfo(np.float32).eps * (np.abs(U.host(x.contiguous())).astype(np.float64) @ np.abs(U.host(w)).astype(np.float64))
    assert (np.abs(U.host(r.contiguous()) - want) <= tol).all()
    keep = torch.ones(24, dtype=torch.bool)
    keep[4:4 + n_out] = False
    assert float(rw[:, keep.cuda()].abs().max()) == 0.0      # nothing outside the block was written
    g = rand((rows, n_out), 13)
    wg = torch.empty(n_in, n_out, dtype=torch.complex64, device="cuda")
    ws1, nbytes1 = cabi.mix_workspace(1, rows, n_in, n_out, "cuda")
    cabi.check(L.gelib_hip_part_mix_channels_wgrad(wg.data_ptr(), x.data_ptr(), g.data_ptr(), rows, n_in, n_out, 64, n_out,
                                                   ws1.data_ptr(), nbytes1, None))
    hx, hg = U.host(x.contiguous()).astype(np.complex128), U.host(g).astype(np.complex128)
    assert (np.abs(U.host(wg) - hx.conj().T @ hg) <= 1e-6 + 4 * np.finfo(np.float32).eps * (np.abs(hx).T @ np.abs(hg))).all()


def test_mix_channels_workspace_is_the_callers(cabi):
    """The library allocates nothing for these calls: without a workspace, or with one that is too small or misaligned,
    they return status 13 and launch nothing."""
    rows, n_in, n_out = 64, 32, 16
    x, w = rand((rows, n_in), 21), rand((n_in, n_out), 22)
    r = torch.full((rows, n_out), 5.0, dtype=torch.complex64, device="cuda")
    L = cabi.lib()
    need = int(L.gelib_hip_part_mix_workspace_bytes(0, rows, n_in, n_out))
    assert need > 0 and int(L.gelib_hip_part_mix_workspace_bytes(1, rows, n_in, n_out)) > 0
    assert int(L.gelib_hip_part_mix_workspace_bytes(0, 0, n_in, n_out)) == 0
    ws = torch.empty(need + 16, dtype=torch.uint8, device="cuda")
    call = lambda p, n: L.gelib_hip_part_mix_channels(r.data_ptr(), x.data_ptr(), w.data_ptr(), rows, n_in, n_out,
                                                      n_out, n_in, 0, p, n, None)
    assert call(None, 0) == 13
    assert call(ws.data_ptr(), 16 * n_in * n_out - 16) == 13      # less than the packed matrix itself
    assert call(ws.data_ptr() + 4, need) == 13
    g = rand((rows, n_out), 23)
    wg = torch.empty(n_in, n_out, dtype=torch.complex64, device="cuda")
    assert L.gelib_hip_part_mix_channels_wgrad(wg.data_ptr(), x.data_ptr(), g.data_ptr(), rows, n_in, n_out, n_in, n_out,
                                               None, 0, None) == 13
    torch.cuda.synchronize()
    assert float((r - 5.0).abs().max()) == 0.0
    assert call(ws.data_ptr(), need) == 0
    torch.cuda.synchronize()
    assert float((r - 5.0).abs().max()) > 0.0
