"""The entry points inside a captured HIP graph: product forward and backward, channel mixing (workspace from the
caller, and the variant that allocates nothing) and the fused product -> linear call are recorded once (after an eager
call that uploads the tables of the type signature) and replayed several times on new input values, with eager work and
synchronisations between the replays; every replay must give the bits of the eager calls on the same values."""
import pytest

from tests import gpu_util as U

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def cabi():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from gelib_amd import cabi as c
    c.lib()
    return c


def bits(ts):
    return [t.view(torch.float32).clone() for t in ts]


def test_replays_match_eager_calls(cabi):
    import ctypes
    B, n, n_out = 96, 16, 16
    tau = {l: n for l in range(5)}
    taus = cabi.so3type_product(tau, tau, 4)
    xs = [U.dev(U.seeded(10 + l, B, 2 * l + 1, n)) for l in range(5)]
    ys = [U.dev(U.seeded(20 + l, B, 2 * l + 1, n)) for l in range(5)]
    ws = [U.dev(U.seeded(30 + l, taus[l], n_out, scale=0.05)) for l in range(5)]
    rs = [torch.empty(B, 2 * l + 1, taus[l], dtype=torch.complex64, device="cuda") for l in range(5)]
    xg, yg = [torch.empty_like(t) for t in xs], [torch.empty_like(t) for t in ys]
    mixed = torch.empty(B, 9, n_out, dtype=torch.complex64, device="cuda")
    mixed_static = torch.empty_like(mixed)
    fused = [torch.empty(B, 2 * l + 1, n_out, dtype=torch.complex64, device="cuda") for l in range(5)]
    L = cabi.lib()

    def static_mix(stream):
        rows = B * 9
        cabi.check(L.gelib_hip_part_mix_channels_static(mixed_static.data_ptr(), rs[4].data_ptr(), ws[4].data_ptr(), rows,
                                                        taus[4], n_out, n_out, taus[4], 0, stream))

    def work():
        cabi.so3vec_fwd(rs, xs, ys, accumulate=False)
        cabi.so3vec_bwd(xg, yg, rs, xs, ys, accumulate=False)      # the product itself as the incoming gradient
        cabi.part_mix_channels(mixed, rs[4], ws[4])
        static_mix(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert cabi.so3vec_cg_linear_fwd(fused, xs, ys, ws, accumulate=False)

    outputs = lambda: bits(rs + xg + yg + [mixed, mixed_static] + fused)
    # A backward launch with few cells deals the pairs of a cell to several blocks and adds their sums from a scratch
    # buffer of the library's own; a call that is being recorded gets no such buffer (the graph would keep its address)
    # and runs one block per cell.  The eager calls this test compares with are made the same way, so that the bits agree.
    cabi.set_option("unrolled_bwd_split", 0)
    work()                      # eager: uploads the tables, validates the allocations
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        work()
    torch.cuda.synchronize()
    for k in range(3):
        for l in range(5):      # new values in the buffers the graph reads
            xs[l].copy_(U.dev(U.seeded(100 + 10 * k + l, B, 2 * l + 1, n)))
            ys[l].copy_(U.dev(U.seeded(200 + 10 * k + l, B, 2 * l + 1, n)))
        work()
        torch.cuda.synchronize()
        want = outputs()
        for t in rs + xg + yg + [mixed, mixed_static] + fused:
            t.fill_(7.0)
        junk = torch.randn(1 << 20, device="cuda").sum()      # unrelated eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = outputs()
        assert all(torch.equal(a, b) for a, b in zip(got, want)), "replay %d" % k
        assert bool(torch.isfinite(junk))
    cabi.set_option("unrolled_bwd_split", 1)
    # with the split on, the eager call agrees with the recorded one to rounding
    work()
    torch.cuda.synchronize()
    for a, b in zip(xg + yg, got[5:15]):
        assert torch.allclose(a.view(torch.float32), b, rtol=1e-4, atol=1e-3)


def test_recorded_calls_use_lent_scratch(cabi):
    """With memory lent for the stream (gelib_hip_set_stream_workspace), a recorded call takes the routes an eager call
    takes -- the pairs of a cell dealt to several blocks in a launch with few cells, per-cell gradients and a fixed-order
    sum for an operand shared by the batch -- and replays give the eager bits."""
    B, n = 48, 16
    cabi.set_option("unrolled_bwd_split", 1)
    xs = [U.dev(U.seeded(10 + l, B, 2 * l + 1, n)) for l in range(5)]
    x1 = [U.dev(U.seeded(40 + l, 1, 2 * l + 1, n)) for l in range(5)]
    ys = [U.dev(U.seeded(20 + l, B, 2 * l + 1, n)) for l in range(5)]
    taus = cabi.so3type_product({l: n for l in range(5)}, {l: n for l in range(5)}, 4)
    gs = [U.dev(U.seeded(30 + l, B, 2 * l + 1, taus[l])) for l in range(5)]
    xg, yg = [torch.empty_like(t) for t in xs], [torch.empty_like(t) for t in ys]
    xg1, yg1 = [torch.empty_like(t) for t in x1], [torch.empty_like(t) for t in ys]
    stream = torch.cuda.Stream()
    lent = torch.empty(64 << 20, dtype=torch.uint8, device="cuda")
    cabi.set_stream_workspace(lent, stream)
    paths = []

    def work():
        cabi.so3vec_bwd(xg, yg, gs, xs, ys, accumulate=False)
        paths.append(cabi.last_path())
        cabi.so3vec_bwd(xg1, yg1, gs, x1, ys, accumulate=False)      # x shared by the batch
        paths.append(cabi.last_path())

    try:
        with torch.cuda.stream(stream):
            work()
        torch.cuda.synchronize()
        want = bits(xg + yg + xg1 + yg1)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            work()
        torch.cuda.synchronize()
        assert paths == [2, 2, 2, 2]          # the unrolled kernels, also for the shared operand, also while recording
        for k in range(2):
            for t in xg + yg + xg1 + yg1:
                t.fill_(7.0)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert all(torch.equal(a, b) for a, b in zip(bits(xg + yg + xg1 + yg1), want)), "replay %d" % k
        # without the loan a recorded call takes the scratch-free routes and still agrees to rounding (an eager call on
        # that route first: it uploads the per-triple tables of the shape-agnostic kernels, which a recorded call cannot)
        cabi.set_stream_workspace(None, stream)
        cabi.set_option("bcast_reduce", 0)
        with torch.cuda.stream(stream):
            cabi.so3vec_bwd(xg1, yg1, gs, x1, ys, accumulate=False)
        torch.cuda.synchronize()
        cabi.set_option("bcast_reduce", 1)
        paths.clear()
        graph2 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph2, stream=stream):
            work()
        torch.cuda.synchronize()
        assert paths == [2, 1]
        graph2.replay()
        torch.cuda.synchronize()
        for a, b in zip(bits(xg + yg + xg1 + yg1), want):
            assert torch.allclose(a, b, rtol=1e-4, atol=1e-3)
    finally:
        cabi.set_option("bcast_reduce", 1)
        cabi.set_stream_workspace(None, stream)
