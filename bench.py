#!/usr/bin/env python3
"""Benchmark of the fused SO3vec CGproduct path on one MI355X.

One "step" = one forward pass (all (l1,l2,l) triples, one launch) plus one backward pass (both gradients, one
launch) over a batch of synthetic complex64 N(0,1) inputs that already sit in HBM.  The default workload is the
headline configuration: L=4, 16 channels per part, batch 32768, product capped at l<=4 (65 triples).

Prints ONE JSON line: samples/s (whole job), the roofline of the dominant kernel from HIP-event timings taken
inside this run, and a CPU baseline (the oracle's loop-order-faithful float32 restatement of the reference's CPU
path, timed here on one host core over a batch slice; the GPU result for that slice is checked against it, every
component, and the run exits with status 3 if one fails).  After the headline, the default run times the other
configurations of the baseline list the same way and reports one record each under config.all_configs.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12  # B/s, MI355X HBM3E

TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")


def kernel_sources_digest():
    """sha256 over the kernel sources (file names and contents, sorted): what a traffic measurement belongs to."""
    import hashlib
    d = os.path.join(ROOT, "gelib_amd", "csrc")
    h = hashlib.sha256()
    for fn in sorted(os.listdir(d)):
        if fn.endswith((".hip", ".h", ".cpp")) or fn == "Makefile":
            h.update(fn.encode())
            with open(os.path.join(d, fn), "rb") as f:
                h.update(f.read())
    return h.hexdigest()


def measured_traffic(name, key):
    """HBM bytes per launch from profiles/hbm_traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, two runs, each
    scaled by what the counter reads for a plain 1 GiB copy), or None when the kernel sources have changed since the
    counters were read: a stale figure is not printed."""
    try:
        with open(TRAFFIC_FILE) as f:
            t = json.load(f)
    except (OSError, ValueError):
        return None
    rec = t.get("workloads", {}).get(name)
    if not rec or rec.get("sources_sha256") != kernel_sources_digest():
        return None
    return rec.get(key)


WORKLOADS = {
    # name: (kind, B, tau_x, tau_y, maxl, diag)
    "so3vec_cg_L4_tau16_B32768_maxl4": ("vec", 32768, {l: 16 for l in range(5)}, {l: 16 for l in range(5)}, 4, False),
    "so3vec_cg_L4_tau16_B32768_uncapped": ("vec", 32768, {l: 16 for l in range(5)}, {l: 16 for l in range(5)}, -1, False),
    # kind "part": ONE triple through the part-level entry points (forward; backward = back0 + back1, two calls, as
    # the reference's SO3part operator makes them); the fifth field is the l of the triple
    "so3part_cg_2x3to4_n32_B65536": ("part", 65536, {2: 32}, {3: 32}, 4, False),
    "so3vec_cg_l2_x_l3_n32_B65536_maxl4": ("vec", 65536, {2: 32}, {3: 32}, 4, False),   # the same pair into l = 1..4
    "so3vec_diagcg_L6_n64_B131072": ("vec", 131072, {l: 64 for l in range(7)}, {l: 64 for l in range(7)}, 6, True),
    "so3part_cg_10x10_all_l_n8_B16384": ("vec", 16384, {10: 8}, {10: 8}, -1, False),
    "so3vec_diagcg_L4_n64_B131072": ("vec", 131072, {l: 64 for l in range(5)}, {l: 64 for l in range(5)}, 4, True),
    "so3vec_diagcg_L4_n16_B524288": ("vec", 524288, {l: 16 for l in range(5)}, {l: 16 for l in range(5)}, 4, True),
    "so3vec_cg_L6_tau8_B16384_maxl6": ("vec", 16384, {l: 8 for l in range(7)}, {l: 8 for l in range(7)}, 6, False),
    "so3vec_cg_L6_tau8_B16384_uncapped": ("vec", 16384, {l: 8 for l in range(7)}, {l: 8 for l in range(7)}, -1, False),
    "so3vec_cg_L4_tau4_B524288_maxl4": ("vec", 524288, {l: 4 for l in range(5)}, {l: 4 for l in range(5)}, 4, False),
    "so3vec_cg_L2_tau64_B8192_maxl2": ("vec", 8192, {l: 64 for l in range(3)}, {l: 64 for l in range(3)}, 2, False),
    "so3vec_diagcg_L4_n64_B131072_uncapped": ("vec", 131072, {l: 64 for l in range(5)}, {l: 64 for l in range(5)}, -1, True),
    "so3part_cg_1x1to1_n16_B1024": ("part", 1024, {1: 16}, {1: 16}, 1, False),
    "so3vec_cg_l8l10_x_l9l10_tau4_B32768_maxl12": ("vec", 32768, {8: 4, 10: 4}, {9: 4, 10: 4}, 12, False),
}
HEADLINE = "so3vec_cg_L4_tau16_B32768_maxl4"
# the configurations of the baseline list other than the headline, with the size of the CPU slice each is checked on
OTHER_CONFIGS = [("so3part_cg_1x1to1_n16_B1024", 1024), ("so3part_cg_2x3to4_n32_B65536", 512),
                 ("so3vec_diagcg_L6_n64_B131072", 64), ("so3vec_cg_L4_tau16_B32768_uncapped", 256),
                 ("so3part_cg_10x10_all_l_n8_B16384", 64)]
ALIASES = {"cg23": "so3vec_cg_l2_x_l3_n32_B65536_maxl4", "cfg1": "so3part_cg_1x1to1_n16_B1024", "cfg4": "so3vec_cg_L4_tau16_B32768_maxl4", "cfg4u": "so3vec_cg_L4_tau16_B32768_uncapped",
           "cfg2": "so3part_cg_2x3to4_n32_B65536", "cfg3": "so3vec_diagcg_L6_n64_B131072",
           "cfg5": "so3part_cg_10x10_all_l_n8_B16384", "diag4": "so3vec_diagcg_L4_n64_B131072",
           "diag4n16": "so3vec_diagcg_L4_n16_B524288", "cg6": "so3vec_cg_L6_tau8_B16384_maxl6", "cg6u": "so3vec_cg_L6_tau8_B16384_uncapped",
           "diag4u": "so3vec_diagcg_L4_n64_B131072_uncapped", "cg2n64": "so3vec_cg_L2_tau64_B8192_maxl2",
           "cg4n4": "so3vec_cg_L4_tau4_B524288_maxl4", "cg10m": "so3vec_cg_l8l10_x_l9l10_tau4_B32768_maxl12"}


def out_type(tx, ty, maxl, diag):
    tau = {}
    for l1, n1 in sorted(tx.items()):
        for l2, n2 in sorted(ty.items()):
            for l in range(abs(l1 - l2), l1 + l2 + 1):
                if maxl < 0 or l <= maxl:
                    tau[l] = tau.get(l, 0) + (n1 if diag else n1 * n2)
    return dict(sorted(tau.items()))


def algorithmic_bytes(B, tx, ty, tr):
    """Every operand read once and every result written once, complex64 = 8 B."""
    X = 8 * B * sum((2 * l + 1) * n for l, n in tx.items())
    Y = 8 * B * sum((2 * l + 1) * n for l, n in ty.items())
    R = 8 * B * sum((2 * l + 1) * n for l, n in tr.items())
    return X + Y + R, R + 2 * X + 2 * Y


def seeded_parts(torch, seed, B, tau, device, scale=1.0):
    parts = []
    for l, n in sorted(tau.items()):
        g = torch.Generator(device=device).manual_seed(seed + l)
        t = torch.randn(B, 2 * l + 1, n, 2, generator=g, device=device, dtype=torch.float32)
        parts.append(torch.view_as_complex(t) * scale if scale != 1.0 else torch.view_as_complex(t))
    return parts


def cpu_slice(torch, xs, ys, gs, rs, xgs, ygs, maxl, diag, nsample, single_core, part=False):
    """The oracle on the first `nsample` samples: timed (one thread, if single_core, and with the batch loop split over
    the host's cores, which is what the reference's MultiLoop would do) and used as the checker of the GPU results for
    that slice.  Every real component is held to the parity rules of tests/gpu_util.py (gate, or one of the two stated
    rules for sums that nearly cancel); the fractions that needed each rule are reported."""
    import numpy as np
    from oracle import cg_oracle as ora
    from tests import gpu_util as U
    hx = [t[:nsample].cpu().numpy() for t in xs]
    hy = [t[:nsample].cpu().numpy() for t in ys]
    hg = [t[:nsample].cpu().numpy() for t in gs]
    ora.lib()
    nth = max(1, min(16, ora.max_threads(), os.cpu_count() or 1))
    dt1 = None
    if part:   # one triple: maxl is its l
        def both(g, x, y, nthreads):
            r = ora.cg_fwd(x[0], y[0], maxl, diag, nthreads)
            a, b = ora.cg_bwd(g[0], x[0], y[0], diag, nthreads)
            return [r], [a], [b]
        if single_core:
            t0 = time.perf_counter()
            both(hg, hx, hy, 1)
            dt1 = time.perf_counter() - t0
        t0 = time.perf_counter()
        r, xg, yg = both(hg, hx, hy, nth)
        dt_all = time.perf_counter() - t0
        r64, xg64, yg64 = both(U.c128(hg), U.c128(hx), U.c128(hy), nth)
        Sr, Sx, Sy = ([a] for a in ora.cg_term_sums(hg[0], hx[0], hy[0], maxl, diag, nth))
    else:
        if single_core:
            t0 = time.perf_counter()
            ora.vec_fwd(hx, hy, maxl, diag, nthreads=1)
            ora.vec_bwd(hg, hx, hy, diag, nthreads=1)
            dt1 = time.perf_counter() - t0
        t0 = time.perf_counter()
        r = ora.vec_fwd(hx, hy, maxl, diag, nthreads=nth)
        xg, yg = ora.vec_bwd(hg, hx, hy, diag, nthreads=nth)
        dt_all = time.perf_counter() - t0
        r64 = ora.vec_fwd(U.c128(hx), U.c128(hy), maxl, diag, nthreads=nth)
        xg64, yg64 = ora.vec_bwd(U.c128(hg), U.c128(hx), U.c128(hy), diag, nthreads=nth)
        Sr = ora.vec_fwd_term_sums(hx, hy, maxl, diag, nthreads=nth)
        Sx, Sy = ora.vec_bwd_term_sums(hg, hx, hy, diag, nthreads=nth)

    def merge(gpu_parts, c32, c64, S):
        tot = {"components": 0, "outside_gate": 0.0, "cpu_f32_outside_gate_of_f64": 0.0, "by_rule_B": 0.0,
               "by_rule_C": 0.0, "rejected": 0, "max_err_over_rule_C_bound": 0.0, "max_gate_excess": 0.0,
               "outside_gate_complex": 0.0, "max_err_vs_f64": {"gpu": 0.0, "cpu_f32": 0.0}}
        elements = 0
        for t, b, c, s in zip(gpu_parts, c32, c64, S):
            a = t[:nsample].cpu().numpy()
            rep = U.parity_counts(a, b, c, s)
            n = rep["components"]
            for k in ("outside_gate", "cpu_f32_outside_gate_of_f64", "by_rule_B", "by_rule_C"):
                tot[k] += rep[k] * n
            tot["components"] += n
            tot["rejected"] += rep["rejected"]
            # the gate read per complex element: |gpu - cpu| <= 1e-6 + 1e-5 |cpu| on the moduli
            tot["outside_gate_complex"] += float((np.abs(a - b) > U.ATOL + U.RTOL * np.abs(b)).sum())
            elements += a.size
            tot["max_err_over_rule_C_bound"] = max(tot["max_err_over_rule_C_bound"], rep["max_err_over_rule_C_bound"])
            tot["max_gate_excess"] = max(tot["max_gate_excess"], U.gate_excess(a, b))
            tot["max_err_vs_f64"]["gpu"] = max(tot["max_err_vs_f64"]["gpu"], U.max_abs_err(a, c))
            tot["max_err_vs_f64"]["cpu_f32"] = max(tot["max_err_vs_f64"]["cpu_f32"], U.max_abs_err(b, c))
        for k in ("outside_gate", "cpu_f32_outside_gate_of_f64", "by_rule_B", "by_rule_C"):
            tot[k] /= max(1, tot["components"])
        tot["outside_gate_complex"] /= max(1, elements)
        return tot

    fwd = merge(rs, r, r64, Sr)
    bwd = merge(xgs + ygs, xg + yg, xg64 + yg64, Sx + Sy)
    parity = {"ok": fwd["rejected"] == 0 and bwd["rejected"] == 0, "samples": nsample, "fwd": fwd, "bwd": bwd,
              "rules": "per real component: A |gpu-cpu| <= 1e-6 + 1e-5|cpu|; else B (cpu_f32 itself outside that gate "
                       "of float64 and |gpu-f64| <= |cpu-f64|); else C |gpu-f64| <= 1e-6 + 2*eps32*sum|terms|; "
                       "outside_gate = fraction not passing A, rejected = components passing none; "
                       "outside_gate_complex = fraction of complex elements with |gpu-cpu| > 1e-6 + 1e-5|cpu| (moduli)"}
    return {"single_core_s": dt1, "all_cores_s": dt_all, "cores": nth, "parity": parity}


AUX_WORKLOADS = ("spharm_l4_n16_B1048576", "gather_l2_n16_cells262144_deg8", "linear_l4_3840to16_B32768")


def aux_bench(torch, args, name):
    """The kernels either side of the product: the producer of y (spherical harmonics), the sum of cells that precedes
    it in message passing (gather), and the linear layer that consumes it (the l = 4 part of the L = 4 product, 3840
    channels, mixed down to 16: forward, gradient of the part, gradient of the matrix).  Same JSON shape; a step is one
    launch (three for the linear layer)."""
    import numpy as np
    from gelib_amd import cabi
    from oracle import cg_oracle as ora
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(77)
    if name.startswith("spharm"):
        l, n, B = 4, 16, args.batch or 1048576
        X = torch.randn(B, 3, n, generator=g).to(dev)
        r = torch.empty(B, 2 * l + 1, n, dtype=torch.complex64, device=dev)
        step = lambda: cabi.so3part_spharm(r, X, accumulate=False)
        nbytes, units, unit = B * n * (12 + 8 * (2 * l + 1)), B * n, "vectors/s"
        ns = min(B, 65536)

        def cpu():
            t0 = time.perf_counter()
            want = ora.spharm(l, X[:ns].cpu().numpy())
            return ns * n / (time.perf_counter() - t0), want, r[:ns].cpu().numpy()
        sample = "first %d of the batch" % ns
        tol = dict(rtol=1e-5, atol=1e-6)
    elif name.startswith("linear"):
        l, n_in, n_out, B = 4, 3840, 16, args.batch or 32768
        gd = torch.Generator(device=dev).manual_seed(78)
        X = torch.view_as_complex(torch.randn(B, 2 * l + 1, n_in, 2, device=dev, generator=gd))
        G = torch.view_as_complex(torch.randn(B, 2 * l + 1, n_out, 2, device=dev, generator=gd))
        W = torch.view_as_complex(torch.randn(n_in, n_out, 2, device=dev, generator=gd))
        r = torch.empty(B, 2 * l + 1, n_out, dtype=torch.complex64, device=dev)
        xg = torch.empty_like(X)
        wg = torch.empty_like(W)

        def step():
            cabi.part_mix_channels(r, X, W)
            cabi.part_mix_channels(xg, G, W, adjoint=True)
            cabi.part_mix_channels_wgrad(wg, X, G)
        rows = B * (2 * l + 1)
        # x is read twice and its gradient written once; the narrow tensors and the matrix are read or written once
        # per kernel that touches them
        nbytes = 8 * (3 * rows * n_in + 3 * rows * n_out + 3 * n_in * n_out)
        units, unit = B, "samples/s"
        ns = min(B, 256)

        def cpu():
            hx, hw = X[:ns].cpu().numpy(), W.cpu().numpy()
            hg = G[:ns].cpu().numpy()
            t0 = time.perf_counter()
            want = hx @ hw
            _ = hg @ hw.conj().T
            _ = hx.reshape(-1, n_in).conj().T @ hg.reshape(-1, n_out)
            return ns / (time.perf_counter() - t0), want, r[:ns].cpu().numpy()
        sample = "first %d samples, numpy complex64 matmuls (what the reference's torch.matmul does on the host)" % ns
        tol = dict(rtol=1e-4, atol=2e-3)   # sums of 7680 float32 terms of size 1
    else:
        l, n, N, deg = 2, 16, args.batch or 262144, 8
        rng = np.random.default_rng(5)
        src = rng.integers(0, N, N * deg).astype(np.int32)
        tgt = rng.integers(0, N, N * deg).astype(np.int32)
        gm = cabi.GatherMap(src.tolist(), tgt.tolist(), N, N)
        X = torch.view_as_complex(torch.randn(1, N, 2 * l + 1, n, 2, generator=g)).to(dev)
        r = torch.empty_like(X)
        step = lambda: cabi.part_gather(r, X, gm, 1, accumulate=False)
        cell = 8 * (2 * l + 1) * n
        nbytes, units, unit = (N * deg + N) * cell, N, "cells/s"   # every pair reads one cell, every target is written once

        def cpu():
            x = X.cpu().numpy()
            t0 = time.perf_counter()
            want = ora.gather(x, src, tgt, N, 1)
            return N / (time.perf_counter() - t0), want, r.cpu().numpy()
        sample = "the whole map (%d pairs), numpy slice adds" % (N * deg)
        tol = dict(rtol=0, atol=0)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms = e0.elapsed_time(e1) / args.steps
    out = {"metric": name.split("_")[0] + " " + unit, "value": units / (wall / args.steps), "unit": unit, "n_gpus": 1,
           "steps": args.steps, "warmup": args.warmup, "ms_per_step": wall * 1e3 / args.steps, "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic", "config": {"workload": name},
           "roofline": {"bound": "hbm", "kernel": name.split("_")[0], "achieved": nbytes / (ms * 1e-3) / 1e9,
                        "peak": HBM_PEAK / 1e9, "unit": "GB/s", "frac": nbytes / (ms * 1e-3) / HBM_PEAK,
                        "traffic": None if args.batch else measured_traffic(name, "step"),
                        "algorithmic_bytes_per_launch": nbytes}}
    if not args.no_cpu:
        rate, want, got = cpu()
        out["cpu_baseline"] = {"value": rate, "unit": unit, "cores": 1, "kind": "port", "sample": sample}
        out["parity"] = {"ok": bool(np.allclose(got, want, **tol))}
    print(json.dumps(out))


FUSED_WORKLOAD = "so3vec_cg_linear_L4_tau16_to16_B32768"
MFMA_F32_PEAK = 157.3e12


def fused_linear_bench(torch, args):
    """CGproduct(x, y, maxl = 4) of the headline operands followed by the per-l weight matrices (16 output channels), forward:
    the fused entry point, which never stores the product, timed beside the two-step form (product launch + one
    channel-mixing launch per part) on the same inputs.  The fused kernel is bound by the matrix and vector units, not by
    memory: its roofline record counts the flops of the product (8 per complex multiply-add of a term) and of the mixing
    against the float32 matrix-core peak."""
    import numpy as np
    from gelib_amd import cabi
    dev = torch.device("cuda:0")
    B = args.batch or 32768
    tx = {l: 16 for l in range(5)}
    tr = out_type(tx, tx, 4, False)
    n_out = 16
    xs = seeded_parts(torch, 101, B, tx, dev)
    ys = seeded_parts(torch, 202, B, tx, dev)
    ws = []
    for l, n in tr.items():
        g = torch.Generator(device=dev).manual_seed(303 + l)
        ws.append(torch.view_as_complex(torch.randn(n, n_out, 2, generator=g, device=dev)) / float(n) ** 0.5)
    outs = [torch.empty(B, 2 * l + 1, n_out, dtype=torch.complex64, device=dev) for l in tr]
    outs2 = [torch.empty_like(o) for o in outs]
    prod = [torch.empty(B, 2 * l + 1, n, dtype=torch.complex64, device=dev) for l, n in tr.items()]

    def fused():
        assert cabi.so3vec_cg_linear_fwd(outs, xs, ys, ws, accumulate=False)

    def two_step():
        cabi.so3vec_fwd(prod, xs, ys, accumulate=False)
        for o, p, w in zip(outs2, prod, ws):
            cabi.part_mix_channels(o, p, w)

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps, (time.perf_counter() - t0) / args.steps

    fused_ms, fused_wall = timed(fused)
    two_ms, _ = timed(two_step)
    # backward: the bounded-memory entry point (the product and its gradient exist for one chunk of the batch at a time,
    # in an 8 GiB workspace) beside the four separate calls on full-size buffers
    gouts = seeded_parts(torch, 404, B, {l: n_out for l in tr}, dev)
    xg, yg = [torch.empty_like(t) for t in xs], [torch.empty_like(t) for t in ys]
    wg = [torch.empty_like(w) for w in ws]

    def chunked_bwd():
        assert cabi.so3vec_cg_linear_bwd(xg, yg, wg, gouts, xs, ys, ws, accumulate=False, workspace_bytes=8 << 30)

    def four_calls_bwd():
        cabi.so3vec_fwd(prod, xs, ys, accumulate=False)
        for w_g, p, g in zip(wg, prod, gouts):
            cabi.part_mix_channels_wgrad(w_g, p, g)
        for p, g, w in zip(prod, gouts, ws):
            cabi.part_mix_channels(p, g, w, adjoint=True)
        cabi.so3vec_bwd(xg, yg, prod, xs, ys, accumulate=False)

    bwd_ms, _ = timed(chunked_bwd)
    bwd4_ms, _ = timed(four_calls_bwd)
    # terms (m1, m2) of one channel of every (l1, l2, l) block
    terms = sum(1 for l1 in tx for l2 in tx for l in range(abs(l1 - l2), min(l1 + l2, 4) + 1)
                for m in range(-l, l + 1) for m1 in range(-l1, l1 + 1) if abs(m - m1) <= l2)
    flops_product = 8 * terms * 16 * 16 * B
    flops_mix = 8 * sum((2 * l + 1) * n for l, n in tr.items()) * n_out * B
    flops = flops_product + flops_mix
    product_bytes = 8 * B * sum((2 * l + 1) * n for l, n in tr.items())
    out = {"metric": "SO3vec CGproduct -> linear, forward, samples/s at L=4 (fused kernel)", "value": B / fused_wall,
           "unit": "samples/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": fused_wall * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "f32", "data": "synthetic",
           "config": {"workload": FUSED_WORKLOAD, "batch": B, "tau_x": tx, "tau_y": tx, "maxl": 4, "tau_product": tr,
                      "n_out": n_out, "fused_fwd_ms": fused_ms, "two_step_fwd_ms": two_ms,
                      "bwd_bounded_memory_ms": bwd_ms, "bwd_four_calls_full_size_ms": bwd4_ms,
                      "bwd_workspace_bytes": 8 << 30, "fwd_bwd_ms": fused_ms + bwd_ms,
                      "speedup_over_two_step": two_ms / fused_ms,
                      "product_bytes_never_stored": product_bytes,
                      "flops": {"product": flops_product, "mixing": flops_mix}},
           "roofline": {"bound": "mfma", "kernel": "cg_linear_fwd (two launches, one per half of the rows)",
                        "achieved": flops / (fused_ms * 1e-3) / 1e12, "peak": MFMA_F32_PEAK / 1e12, "unit": "TFLOP/s",
                        "frac": flops / (fused_ms * 1e-3) / MFMA_F32_PEAK, "traffic": None,
                        "algorithmic_flops_per_step": flops}}
    if not args.no_cpu:
        from oracle import cg_oracle as ora
        from tests import gpu_util as U
        ns = min(B, 2048)
        hx = [t[:ns].cpu().numpy() for t in xs]
        hy = [t[:ns].cpu().numpy() for t in ys]
        hw = [w.cpu().numpy() for w in ws]
        t0 = time.perf_counter()
        p32 = ora.vec_fwd(hx, hy, 4, False, nthreads=1)
        r32 = [np.matmul(p, w) for p, w in zip(p32, hw)]
        dt = time.perf_counter() - t0
        p64 = ora.vec_fwd(U.c128(hx), U.c128(hy), 4, False, nthreads=1)
        r64 = [np.matmul(p, w.astype(np.complex128)) for p, w in zip(p64, hw)]
        S = [np.matmul(s, (np.abs(w.real) + np.abs(w.imag)).astype(np.float64))
             for s, w in zip(ora.vec_fwd_term_sums(hx, hy, 4, False, 1), hw)]
        reps = [U.parity_counts(o[:ns].cpu().numpy(), a, b, c) for o, a, b, c in zip(outs, r32, r64, S)]
        n = sum(r["components"] for r in reps)
        out["cpu_baseline"] = {"value": ns / dt, "unit": "samples/s", "cores": 1, "kind": "port",
                               "sample": "first %d samples: oracle product, then numpy complex64 matmuls, %.1f s" % (ns, dt)}
        out["parity"] = {"ok": all(r["rejected"] == 0 for r in reps), "samples": ns, "components": n,
                         "outside_gate": sum(r["outside_gate"] * r["components"] for r in reps) / n,
                         "cpu_f32_outside_gate_of_f64": sum(r["cpu_f32_outside_gate_of_f64"] * r["components"] for r in reps) / n,
                         "by_rule_B": sum(r["by_rule_B"] * r["components"] for r in reps) / n,
                         "by_rule_C": sum(r["by_rule_C"] * r["components"] for r in reps) / n,
                         "rejected": sum(r["rejected"] for r in reps),
                         "max_err_over_rule_C_bound": max(r["max_err_over_rule_C_bound"] for r in reps),
                         "two_step_vs_fused_max_abs_diff": max(float((a - b).abs().max()) for a, b in zip(outs, outs2))}
    print(json.dumps(out))
    if "parity" in out and not out["parity"]["ok"]:
        print("bench.py: a fused result on the CPU slice passes none of the parity rules", file=sys.stderr)
        sys.exit(3)


PATH_NAMES = {1: "generic", 2: "unrolled", 3: "staged", 4: "diag6", 5: "onepair", 6: "linear"}


def run_cg_workload(torch, cabi, name, steps, warmup, batch=0, cpu_samples=0, single_core=False, copy_probe=False,
                    fill_reference=False):
    """Forward + backward of one product workload: `warmup` untimed steps, then `steps` steps bracketed by device
    synchronisations (wall clock) with HIP events around each call on the stream the kernels run on; then, outside the
    timed region, the CPU oracle on a slice of the batch as checker and baseline.  Frees its buffers on return."""
    dev = torch.device("cuda:0")
    kind, B, tx, ty, maxl, diag = WORKLOADS[name]
    if batch:
        B = batch
    tr = out_type(tx, ty, maxl, diag)
    part = kind == "part"
    if part:
        tr = {maxl: tr[maxl]}
    fwd_bytes, bwd_bytes = algorithmic_bytes(B, tx, ty, tr)
    scale_y = 1e-3 if "10x10" in name else 1.0
    xs = seeded_parts(torch, 1004, B, tx, dev)
    ys = seeded_parts(torch, 2004, B, ty, dev, scale_y)
    gs = seeded_parts(torch, 3004, B, tr, dev)
    rs = [torch.empty(B, 2 * l + 1, n, dtype=torch.complex64, device=dev) for l, n in tr.items()]
    xgs = [torch.empty_like(t) for t in xs]
    ygs = [torch.empty_like(t) for t in ys]

    def fwd():
        if part:
            cabi.so3part_cg_fwd(rs[0], xs[0], ys[0], 0, accumulate=False)
        else:
            cabi.so3vec_fwd(rs, xs, ys, accumulate=False, diag=diag)

    def bwd():   # for one triple too: both gradients from one pass over g, as gelib_amd.SO3part.CGproduct's backward does
        cabi.so3vec_bwd(xgs, ygs, gs, xs, ys, accumulate=False, diag=diag)

    def bwd_two_calls():   # the reference's form: back0 and back1, each reading g
        cabi.so3part_cg_back0(xgs[0], gs[0], ys[0], 0, accumulate=False)
        cabi.so3part_cg_back1(ygs[0], gs[0], xs[0], 0, accumulate=False)

    if copy_probe:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)   # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst
    for _ in range(warmup):
        fwd()
        bwd()
    torch.cuda.synchronize()
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    t0 = time.perf_counter()
    for k in range(steps):
        ev[k][0].record()
        fwd()
        ev[k][1].record()
        bwd()
        ev[k][2].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    path_bwd = cabi.last_path()
    fwd_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / steps
    bwd_ms = sum(e[1].elapsed_time(e[2]) for e in ev) / steps
    fwd()
    path_fwd = cabi.last_path()
    torch.cuda.synchronize()
    full = B == WORKLOADS[name][1]
    rec = {"workload": name, "batch": B, "tau_x": {str(k): v for k, v in tx.items()},
           "tau_y": {str(k): v for k, v in ty.items()}, "maxl": maxl, "diag": diag,
           "entry_points": ("gelib_hip_so3part_cg_fwd; gelib_hip_so3vec_cg_bwd on one-part vectors (both gradients from "
                            "one pass over g)") if part else "gelib_hip_so3vec_cg_fwd; gelib_hip_so3vec_cg_bwd",
           "triples": sum(1 for l1 in tx for l2 in ty for l in range(abs(l1 - l2), l1 + l2 + 1) if l in tr),
           "kernel_path": {"fwd": PATH_NAMES.get(path_fwd, str(path_fwd)), "bwd": PATH_NAMES.get(path_bwd, str(path_bwd))},
           "timed_steps": steps, "ms_per_step_wall": wall * 1e3 / steps, "samples_per_s": B / (wall / steps),
           "fwd_ms": fwd_ms, "bwd_ms": bwd_ms,
           "fwd_ms_min": min(e[0].elapsed_time(e[1]) for e in ev), "bwd_ms_min": min(e[1].elapsed_time(e[2]) for e in ev),
           "fwd_algorithmic_bytes": fwd_bytes, "bwd_algorithmic_bytes": bwd_bytes,
           "fwd_GBps": fwd_bytes / (fwd_ms * 1e-3) / 1e9, "bwd_GBps": bwd_bytes / (bwd_ms * 1e-3) / 1e9,
           "fwd_frac_of_peak": fwd_bytes / (fwd_ms * 1e-3) / HBM_PEAK,
           "bwd_frac_of_peak": bwd_bytes / (bwd_ms * 1e-3) / HBM_PEAK,
           "fwd_bwd_GBps": (fwd_bytes + bwd_bytes) / ((fwd_ms + bwd_ms) * 1e-3) / 1e9,
           "fwd_bwd_frac_of_peak": (fwd_bytes + bwd_bytes) / ((fwd_ms + bwd_ms) * 1e-3) / HBM_PEAK,
           "fwd_traffic_bytes": measured_traffic(name, "so3vec_fwd") if full else None,
           "bwd_traffic_bytes": measured_traffic(name, "so3vec_bwd") if full else None}
    if part:
        # the two part-level calls of the reference's operator, timed after the main loop (their results are the same
        # gradients; the CPU slice below checks what they left in the buffers)
        bwd_two_calls()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(steps):
            bwd_two_calls()
        b.record()
        torch.cuda.synchronize()
        rec["bwd_back0_plus_back1_ms"] = a.elapsed_time(b) / steps
        rec["bwd_back0_plus_back1_algorithmic_bytes"] = 2 * fwd_bytes
    if cpu_samples:
        ns = min(cpu_samples, B)
        c = cpu_slice(torch, xs, ys, gs, rs, xgs, ygs, maxl, diag, ns, single_core, part)
        rec["parity"] = c["parity"]
        rec["cpu"] = {"samples": ns, "cores": c["cores"], "all_cores_samples_per_s": ns / c["all_cores_s"],
                      "single_core_samples_per_s": ns / c["single_core_s"] if c["single_core_s"] else None,
                      "single_core_s": c["single_core_s"]}
    if fill_reference:
        # What a plain streaming kernel reaches on these very buffers (outside the timed region): torch's fill over the
        # product parts.  Write bandwidth on this GPU depends on where a buffer lies in memory (about 5.6 or 6.6 TB/s
        # for one and the same kernel), so this is the yardstick beside the nominal peak.
        def timed(fn):
            fn()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            torch.cuda.synchronize()
            return a.elapsed_time(b) * 1e-3
        rbytes = sum(t.numel() * 8 for t in rs)
        rec["streaming_reference"] = {"torch_fill_of_product_GBps": rbytes / timed(lambda: [t.fill_(1.0) for t in rs]) / 1e9}
    del xs, ys, gs, rs, xgs, ygs
    torch.cuda.empty_cache()
    return rec


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="cfg4")
    ap.add_argument("--batch", type=int, default=0, help="override the batch size (debugging only)")
    ap.add_argument("--cpu-samples", type=int, default=2048)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--only", action="store_true",
                    help="time the named workload alone (the default run also times the other configurations of the "
                         "baseline list and reports them under config.all_configs)")
    ap.add_argument("--generic", action="store_true", help="force the shape-agnostic kernels")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="library tuning option (gelib_hip_set_option), may be repeated")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one plain 1 GiB device copy (reference dispatch for hardware-counter calibration)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; the path shards along the batch with no exchange step, "
              "so --gpus N>1 has nothing to measure here", file=sys.stderr)
        sys.exit(2)

    import torch
    from gelib_amd import cabi
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    cabi.lib()
    cabi.set_option("force_generic", int(args.generic))
    for kv in args.option:
        k, v = kv.split("=")
        cabi.set_option(k, int(v))
    name = ALIASES.get(args.workload, args.workload)
    if name in ("fused_linear", FUSED_WORKLOAD):
        return fused_linear_bench(torch, args)
    aux = [w for w in AUX_WORKLOADS if w == name or w.split("_")[0] == name]
    if aux:
        return aux_bench(torch, args, aux[0])

    rec = run_cg_workload(torch, cabi, name, args.steps, args.warmup, args.batch,
                          0 if args.no_cpu else args.cpu_samples, single_core=True, copy_probe=args.copy_probe,
                          fill_reference=True)
    if rec["bwd_ms"] >= rec["fwd_ms"]:
        dom, dom_ms, dom_bytes, traffic = "so3vec_bwd", rec["bwd_ms"], rec["bwd_algorithmic_bytes"], rec["bwd_traffic_bytes"]
    else:
        dom, dom_ms, dom_bytes, traffic = "so3vec_fwd", rec["fwd_ms"], rec["fwd_algorithmic_bytes"], rec["fwd_traffic_bytes"]
    achieved = dom_bytes / (dom_ms * 1e-3) / 1e9
    parity = rec.pop("parity", None)
    cpu = rec.pop("cpu", None)
    out = {
        "metric": "SO3vec CGproduct fwd+bwd samples/s at L=4; achieved HBM GB/s vs peak",
        "value": rec["samples_per_s"],
        "unit": "samples/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": rec["ms_per_step_wall"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": rec,
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": achieved, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": achieved * 1e9 / HBM_PEAK, "traffic": traffic,
                     "algorithmic_bytes_per_launch": dom_bytes},
    }
    ok = True
    if cpu:
        out["cpu_baseline"] = {"value": cpu["single_core_samples_per_s"], "unit": "samples/s", "cores": 1, "kind": "port",
                               "sample": "first %d samples of the same batch, fwd+bwd, %.1f s" % (cpu["samples"], cpu["single_core_s"]),
                               "all_cores": {"value": cpu["all_cores_samples_per_s"], "unit": "samples/s", "cores": cpu["cores"]}}
        out["parity"] = parity
        ok = ok and parity["ok"]
    if name == HEADLINE and not args.only and not args.batch and not args.generic:
        # the other configurations of the baseline list, each timed the same way (HIP events, >= 10 timed steps) and
        # checked on a CPU slice; outside the headline's timed region
        others = []
        for wl, ns in OTHER_CONFIGS:
            r = run_cg_workload(torch, cabi, wl, max(10, args.steps), 3, 0, 0 if args.no_cpu else ns)
            ok = ok and r.get("parity", {}).get("ok", True)
            others.append(r)
        out["config"]["all_configs"] = others
    print(json.dumps(out))
    if not ok:
        print("bench.py: a GPU result on the CPU slice passes none of the parity rules (see \"parity\")", file=sys.stderr)
        sys.exit(3)


if __name__ == "__main__":
    main()
