"""Helpers shared by the GPU parity tests: seeded inputs, host<->device copies and the parity gate."""
import numpy as np

RTOL = 1e-5   # parity gate of the CG product path: |gpu - cpu| <= ATOL + RTOL * |cpu| per real component
ATOL = 1e-6


def seeded(seed, *shape, scale=1.0):
    """complex64 with iid N(0,1) real and imaginary parts from a fixed seed (same bits on CPU and GPU)."""
    import torch
    g = torch.Generator().manual_seed(seed)
    re = torch.randn(*shape, generator=g, dtype=torch.float32)
    im = torch.randn(*shape, generator=g, dtype=torch.float32)
    return (torch.complex(re, im) * scale).numpy()


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda")


def host(t):
    return t.detach().cpu().numpy()


def components(a):
    a = np.ascontiguousarray(a)
    return a.view(np.float32 if a.dtype == np.complex64 else np.float64)


def gate_excess(got, ref, rtol=RTOL, atol=ATOL):
    """max over components of |got-ref| / (atol + rtol*|ref|); <= 1 means inside the gate."""
    g = components(got).astype(np.float64)
    r = components(ref).astype(np.float64)
    return float(np.max(np.abs(g - r) / (atol + rtol * np.abs(r)))) if g.size else 0.0


def max_err(got, exact):
    g = components(got).astype(np.float64)
    e = components(np.asarray(exact, dtype=np.complex128))
    return float(np.max(np.abs(g - e))) if g.size else 0.0


def assert_parity(got, cpu32, exact64, what, slack=1.0):
    """Inside the gate against the float32 CPU path.  Where a long float32 sum makes the CPU path itself
    deviate from the exact (float64) answer by more than the gate allows, the GPU result must instead be at
    least as close to the exact answer as the CPU path is (factor `slack`)."""
    ex = gate_excess(got, cpu32)
    if ex <= 1.0:
        return
    e_gpu = max_err(got, exact64)
    e_cpu = max_err(cpu32, exact64)
    assert e_gpu <= slack * e_cpu + ATOL, "%s: gate excess %.2f, gpu err %.3e vs cpu err %.3e" % (what, ex, e_gpu, e_cpu)
