"""The channel-mixing entry point that allocates nothing (gelib_hip_part_mix_channels_static): through the C ABI, against
gelib_hip_part_mix_channels on the same inputs, bit for bit (same kernels, same packed matrix), two calls in a row with
the second one smaller, while torch's allocator statistics and the driver's free-memory figure stay where they were."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def cabi():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from gelib_amd import cabi as c
    L = c.lib()
    # the first call on a device asks the runtime for the address of the array (and, with deferred loading, makes it
    # load the code object): set-up, not part of what the calls below may do
    x, w = rand((4, 2), 1), rand((2, 2), 2)
    r = torch.empty(4, 2, dtype=torch.complex64, device="cuda")
    assert L.gelib_hip_part_mix_channels_static(r.data_ptr(), x.data_ptr(), w.data_ptr(), 4, 2, 2, 2, 2, 0, None) == 0
    torch.cuda.synchronize()
    return c


def rand(shape, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.view_as_complex(torch.randn(*shape, 2, generator=g)).cuda()


def both(cabi, rows, n_in, n_out, adjoint, seed):
    """(result of the entry point with a caller's workspace, result of the one that allocates nothing)"""
    L = cabi.lib()
    x = rand((rows, n_in), seed)
    w = rand((n_out, n_in) if adjoint else (n_in, n_out), seed + 1)
    r_ws = torch.full((rows, n_out), 7.0, dtype=torch.complex64, device="cuda")
    r_st = torch.full((rows, n_out), 9.0, dtype=torch.complex64, device="cuda")
    ws, nbytes = cabi.mix_workspace(0, rows, n_in, n_out, "cuda")
    torch.cuda.synchronize()
    print("static mix: rows %d n_in %d n_out %d adjoint %d" % (rows, n_in, n_out, adjoint), flush=True)
    free0, _ = torch.cuda.mem_get_info()
    reserved0 = torch.cuda.memory_reserved()
    rc = L.gelib_hip_part_mix_channels_static(r_st.data_ptr(), x.data_ptr(), w.data_ptr(), rows, n_in, n_out, n_out,
                                              n_in, int(adjoint), None)
    assert rc == 0, rc
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert torch.cuda.memory_reserved() == reserved0 and free1 == free0      # nothing was allocated on the way
    cabi.check(L.gelib_hip_part_mix_channels(r_ws.data_ptr(), x.data_ptr(), w.data_ptr(), rows, n_in, n_out, n_out,
                                             n_in, int(adjoint), ws.data_ptr(), nbytes, None))
    torch.cuda.synchronize()
    return r_ws, r_st


@pytest.mark.parametrize("adjoint", [False, True])
def test_two_calls_in_a_row_the_second_smaller(cabi, adjoint):
    # the first call fills a large part of the array; the second, smaller one must not see what the first left behind
    a_ws, a_st = both(cabi, 3000, 4352, 16, adjoint, 31) if not adjoint else both(cabi, 3000, 16, 4352, adjoint, 31)
    assert torch.equal(torch.view_as_real(a_ws), torch.view_as_real(a_st))
    b_ws, b_st = both(cabi, 517, 38, 12, adjoint, 41) if not adjoint else both(cabi, 517, 12, 38, adjoint, 41)
    assert torch.equal(torch.view_as_real(b_ws), torch.view_as_real(b_st))
    # and against the exact product, with the tolerance of the channel-mixing tests
    L = cabi.lib()
    rows, n_in, n_out = 200, 64, 48
    x, w = rand((rows, n_in), 51), rand((n_in, n_out), 52)
    r = torch.empty(rows, n_out, dtype=torch.complex64, device="cuda")
    assert L.gelib_hip_part_mix_channels_static(r.data_ptr(), x.data_ptr(), w.data_ptr(), rows, n_in, n_out, n_out,
                                                n_in, 0, None) == 0
    torch.cuda.synchronize()
    hx, hw = x.cpu().numpy().astype(np.complex128), w.cpu().numpy().astype(np.complex128)
    tol = 1e-6 + 4 * np.finfo(np.float32).eps * (np.abs(hx) @ np.abs(hw))
    assert (np.abs(r.cpu().numpy() - hx @ hw) <= tol).all()


def test_sizes_beyond_the_array_are_refused(cabi):
    L = cabi.lib()
    rows, n_in, n_out = 8, 4096, 256            # 16 MiB of packed matrix: twice what the array holds
    assert int(L.gelib_hip_part_mix_workspace_bytes(0, rows, n_in, n_out)) > (8 << 20)
    x, w = rand((rows, n_in), 61), rand((n_in, n_out), 62)
    r = torch.full((rows, n_out), 3.0, dtype=torch.complex64, device="cuda")
    rc = L.gelib_hip_part_mix_channels_static(r.data_ptr(), x.data_ptr(), w.data_ptr(), rows, n_in, n_out, n_out, n_in,
                                              0, None)
    assert rc == 14
    assert b"8 MiB" in L.gelib_hip_strerror(14)
    torch.cuda.synchronize()
    assert float((r - 3.0).abs().max()) == 0.0          # nothing was launched
    # the largest size that fits still runs
    n_in, n_out = 2048, 256                             # exactly 8 MiB
    assert int(L.gelib_hip_part_mix_workspace_bytes(0, rows, n_in, n_out)) == (8 << 20)
    x, w = rand((rows, n_in), 63), rand((n_in, n_out), 64)
    r = torch.empty(rows, n_out, dtype=torch.complex64, device="cuda")
    assert L.gelib_hip_part_mix_channels_static(r.data_ptr(), x.data_ptr(), w.data_ptr(), rows, n_in, n_out, n_out, n_in,
                                                0, None) == 0
    torch.cuda.synchronize()
    hx, hw = x.cpu().numpy().astype(np.complex128), w.cpu().numpy().astype(np.complex128)
    assert (np.abs(r.cpu().numpy() - hx @ hw) <= 1e-6 + 4 * np.finfo(np.float32).eps * (np.abs(hx) @ np.abs(hw))).all()
