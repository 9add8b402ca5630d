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


def max_abs_err(got, exact):
    g = components(got).astype(np.float64)
    e = components(np.asarray(exact, dtype=np.complex128))
    return float(np.max(np.abs(g - e))) if g.size else 0.0


EPS32 = float(np.finfo(np.float32).eps)
TERM_SUM_FACTOR = 2.0   # rule C below


def moduli(a):
    """|a| as complex128 with zero imaginary part: the operand form of the oracle's term-sum runs."""
    return np.abs(a).astype(np.complex128)


def c128(parts):
    return [np.asarray(a).astype(np.complex128) for a in parts]


def parity_counts(got, cpu32, exact64, term_sums):
    """Per real component, which rule accepts the GPU value g, given the float32 CPU value c of the reference's loop
    order, the float64 value e of the same loops, and S = the sum of the moduli of the element's terms:

      A  |g - c| <= ATOL + RTOL*|c|                       the parity gate itself;
      B  c itself lies outside that gate around e, and |g - e| <= |c - e|
                                                          (the reference's own float32 sum misses the gate; the GPU
                                                          value is at least as close to the exact one);
      C  |g - e| <= ATOL + TERM_SUM_FACTOR*EPS32*S        (the element nearly cancels, so its gate is narrower than the
                                                          rounding error of ANY float32 evaluation, which follows S and
                                                          not the value; 2*EPS32*S is the bound the reference's own
                                                          float32 results satisfy against float64: measured 1.98 at
                                                          most over every kernel family's test shapes, GPU at most 0.96).

    Every component must be accepted by one of them; nothing is compared in a norm.  Returns the counts."""
    g = components(got).astype(np.float64)
    c = components(cpu32).astype(np.float64)
    e = components(np.asarray(exact64, dtype=np.complex128))
    assert g.shape == c.shape == e.shape, (g.shape, c.shape, e.shape)
    S = np.repeat(np.asarray(term_sums, dtype=np.float64).reshape(-1), 2).reshape(g.shape)
    in_a = np.abs(g - c) <= ATOL + RTOL * np.abs(c)
    cpu_out = np.abs(c - e) > ATOL + RTOL * np.abs(e)
    in_b = ~in_a & cpu_out & (np.abs(g - e) <= np.abs(c - e))
    in_c = ~in_a & ~in_b & (np.abs(g - e) <= ATOL + TERM_SUM_FACTOR * EPS32 * S)
    bad = ~(in_a | in_b | in_c)
    n = max(1, g.size)
    worst = float(np.max(np.abs(g - e) / (ATOL + TERM_SUM_FACTOR * EPS32 * S))) if g.size else 0.0
    return {"components": int(g.size), "outside_gate": float((~in_a).sum() / n),
            "cpu_f32_outside_gate_of_f64": float(cpu_out.sum() / n), "by_rule_B": float(in_b.sum() / n),
            "by_rule_C": float(in_c.sum() / n), "rejected": int(bad.sum()),
            "max_err_over_rule_C_bound": worst,
            "first_rejected": int(np.flatnonzero(bad.reshape(-1))[0]) if bad.any() else -1}


def assert_parity(got, cpu32, exact64, term_sums, what):
    """Every real component must pass rule A, B or C of parity_counts."""
    rep = parity_counts(got, cpu32, exact64, term_sums)
    assert rep["rejected"] == 0, "%s: %s" % (what, rep)
    return rep


def assert_gate(got, cpu32, what=""):
    """Rule A alone: every component inside the parity gate of the float32 CPU value (the forward pass)."""
    ex = gate_excess(got, cpu32)
    assert ex <= 1.0, "%s: gate excess %.3f" % (what, ex)


class VecOracle:
    """All the oracle has to say about one SO3vec product on given inputs: float32 (reference loop order) and float64
    results of forward and backward, and the per-element term sums that rule C of the parity check needs."""

    def __init__(self, xs, ys, maxl, diag, gs=None, gseed=None, nthreads=1):
        from oracle import cg_oracle as ora
        self.xs, self.ys, self.maxl, self.diag = xs, ys, maxl, diag
        nt = nthreads
        self.r32 = ora.vec_fwd(xs, ys, maxl, diag, nt)
        self.r64 = ora.vec_fwd(c128(xs), c128(ys), maxl, diag, nt)
        self.Sr = ora.vec_fwd_term_sums(xs, ys, maxl, diag, nt)
        if gs is None and gseed is not None:
            gs = [seeded(gseed + i, *p.shape) for i, p in enumerate(self.r32)]
        self.gs = gs
        if gs is not None:
            self.set_gradient(gs, nt)

    def set_gradient(self, gs, nthreads=1):
        from oracle import cg_oracle as ora
        xs, ys, diag = self.xs, self.ys, self.diag
        self.gs = gs
        self.xg32, self.yg32 = ora.vec_bwd(gs, xs, ys, diag, nthreads)
        self.xg64, self.yg64 = ora.vec_bwd(c128(gs), c128(xs), c128(ys), diag, nthreads)
        self.Sx, self.Sy = ora.vec_bwd_term_sums(gs, xs, ys, diag, nthreads)

    def check_fwd(self, got_parts, what):
        """Every component under the three rules.  Sums of at most 9 terms (operand l up to 4) sit inside the gate
        itself except for about one component in 10^8 (measured over 24 seeds of the L=4 product), so there at most
        one component, or one in 10^7, may need rule B or C."""
        short = max((a.shape[1] - 1) // 2 for a in list(self.xs) + list(self.ys)) <= 4
        for a, b, c, s in zip(got_parts, self.r32, self.r64, self.Sr):
            rep = assert_parity(a, b, c, s, "fwd " + what)
            if short:
                n = rep["components"]
                assert rep["outside_gate"] * n <= 1 + 1e-7 * n, "fwd %s: %s" % (what, rep)

    def check_bwd(self, got_xg, got_yg, what):
        if got_xg is not None:
            for a, b, c, s in zip(got_xg, self.xg32, self.xg64, self.Sx):
                assert_parity(a, b, c, s, "xg " + what)
        if got_yg is not None:
            for a, b, c, s in zip(got_yg, self.yg32, self.yg64, self.Sy):
                assert_parity(a, b, c, s, "yg " + what)

    def check_bwd_onto(self, got_xg, got_yg, start_xg, start_yg, what):
        """Accumulate mode: the gradients were added onto start_xg / start_yg.  The oracle adds its terms onto copies
        of the same starting values (the reference's add_... semantics); the start is one more term of every sum."""
        from oracle import cg_oracle as ora
        b0, b1 = (ora.DIAG_BACK0, ora.DIAG_BACK1) if self.diag else (ora.CG_BACK0, ora.CG_BACK1)
        for got, start, op, S in ((got_xg, start_xg, b0, self.Sx), (got_yg, start_yg, b1, self.Sy)):
            if got is None:
                continue
            w32 = [np.array(a, dtype=np.complex64) for a in start]
            w64 = c128(start)
            if op == b0:
                ora.vec_op(op, self.gs, w32, self.ys)
                ora.vec_op(op, c128(self.gs), w64, c128(self.ys))
            else:
                ora.vec_op(op, self.gs, self.xs, w32)
                ora.vec_op(op, c128(self.gs), c128(self.xs), w64)
            for a, b, c, s, st in zip(got, w32, w64, S, start):
                assert_parity(a, b, c, s + np.abs(st), what)

    def check_fwd_onto(self, got_parts, start_parts, what):
        """Accumulate mode forward: the product was added onto start_parts."""
        from oracle import cg_oracle as ora
        op = ora.DIAG_FWD if self.diag else ora.CG_FWD
        w32 = [np.array(a, dtype=np.complex64) for a in start_parts]
        w64 = c128(start_parts)
        ora.vec_op(op, w32, self.xs, self.ys)
        ora.vec_op(op, w64, c128(self.xs), c128(self.ys))
        for a, b, c, s, st in zip(got_parts, w32, w64, self.Sr, start_parts):
            assert_parity(a, b, c, s + np.abs(st), "fwd " + what)
