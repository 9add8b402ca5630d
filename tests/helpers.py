"""Independent mathematical helpers for the tests: exact Clebsch-Gordan coefficients (sympy), Wigner-D
matrices from angular-momentum generators (scipy expm), brute-force and einsum products."""
import functools
import json
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@functools.lru_cache(maxsize=None)
def sympy_cg_matrix(l1, l2, l):
    """(2l1+1)x(2l2+1) float64 table of <l1 m1; l2 m2 | l m1+m2> from sympy's exact radicals."""
    from sympy import S
    from sympy.physics.quantum.cg import CG
    out = np.zeros((2 * l1 + 1, 2 * l2 + 1))
    for m1 in range(-l1, l1 + 1):
        for m2 in range(-l2, l2 + 1):
            if abs(m1 + m2) <= l:
                out[m1 + l1, m2 + l2] = float(CG(S(l1), S(m1), S(l2), S(m2), S(l), S(m1 + m2)).doit().evalf(30))
    return out


@functools.lru_cache(maxsize=None)
def golden_cg_tables():
    """Exact-coefficient fixture written by tests/golden/make_cg_tables.py (sympy, 17 significant digits)."""
    with open(os.path.join(GOLDEN, "cg_tables_sympy.json")) as f:
        raw = json.load(f)
    return {tuple(int(v) for v in k.split(",")): np.array(t, dtype=np.float64) for k, t in raw.items()}


def dense_cg_tensor(C, l1, l2, l):
    """W[m1,m2,m] with W[m1,m2,m1+m2]=C[m1,m2] on the valid set, from a (2l1+1)x(2l2+1) table."""
    W = np.zeros((2 * l1 + 1, 2 * l2 + 1, 2 * l + 1))
    for m1 in range(-l1, l1 + 1):
        for m2 in range(-l2, l2 + 1):
            if abs(m1 + m2) <= l:
                W[m1 + l1, m2 + l2, m1 + m2 + l] = C[m1 + l1, m2 + l2]
    return W


def einsum_cg(x, y, C, l, diag=False):
    """complex128 product from a coefficient table; x (B,2l1+1,N1), y (B,2l2+1,N2)."""
    l1 = (x.shape[1] - 1) // 2
    l2 = (y.shape[1] - 1) // 2
    W = dense_cg_tensor(np.asarray(C, dtype=np.float64), l1, l2, l)
    x = x.astype(np.complex128)
    y = y.astype(np.complex128)
    if diag:
        return np.einsum("bic,bjc,ijm->bmc", x, y, W)
    B = max(x.shape[0], y.shape[0])
    r = np.einsum("bic,bjd,ijm->bmcd", x, y, W)
    return r.reshape(B, 2 * l + 1, x.shape[2] * y.shape[2])


def einsum_cg_bwd(g, x, y, C, diag=False):
    """Gradients in the conjugate convention: xg = sum C g conj(y), yg = sum C g conj(x)."""
    l1 = (x.shape[1] - 1) // 2
    l2 = (y.shape[1] - 1) // 2
    l = (g.shape[1] - 1) // 2
    W = dense_cg_tensor(np.asarray(C, dtype=np.float64), l1, l2, l)
    x = x.astype(np.complex128)
    y = y.astype(np.complex128)
    g = g.astype(np.complex128)
    if diag:
        xg = np.einsum("bmc,bjc,ijm->bic", g, y.conj(), W)
        yg = np.einsum("bmc,bic,ijm->bjc", g, x.conj(), W)
        return xg, yg
    B = g.shape[0]
    g4 = g.reshape(B, 2 * l + 1, x.shape[2], y.shape[2])
    xg = np.einsum("bmcd,bjd,ijm->bic", g4, y.conj(), W)
    yg = np.einsum("bmcd,bic,ijm->bjd", g4, x.conj(), W)
    return xg, yg


def brute_cg(x, y, C, l, diag=False):
    """Pure-Python loops straight from the definition (tiny inputs only)."""
    B, M1, N1 = x.shape
    _, M2, N2 = y.shape
    l1, l2 = (M1 - 1) // 2, (M2 - 1) // 2
    r = np.zeros((B, 2 * l + 1, N1 if diag else N1 * N2), dtype=np.complex128)
    for b in range(B):
        for m1 in range(-l1, l1 + 1):
            for m2 in range(-l2, l2 + 1):
                m = m1 + m2
                if abs(m) > l:
                    continue
                for i in range(N1):
                    for j in ([i] if diag else range(N2)):
                        ch = i if diag else i * N2 + j
                        r[b, m + l, ch] += C[m1 + l1, m2 + l2] * complex(x[b, m1 + l1, i]) * complex(y[b, m2 + l2, j])
    return r


def wigner_D(l, alpha, beta, gamma):
    """D^l = exp(-i alpha Jz) exp(-i beta Jy) exp(-i gamma Jz), basis m=-l..l, Condon-Shortley ladder phases."""
    from scipy.linalg import expm
    m = np.arange(-l, l + 1)
    Jz = np.diag(m).astype(np.complex128)
    Jp = np.zeros((2 * l + 1, 2 * l + 1), dtype=np.complex128)
    for k in range(2 * l):
        mm = m[k]
        Jp[k + 1, k] = np.sqrt(l * (l + 1) - mm * (mm + 1))
    Jm = Jp.conj().T
    Jy = (Jp - Jm) / 2j
    return expm(-1j * alpha * Jz) @ expm(-1j * beta * Jy) @ expm(-1j * gamma * Jz)


def rotate(part, angles):
    l = (part.shape[-2] - 1) // 2
    return wigner_D(l, *angles) @ part.astype(np.complex128)


def randc(rng, *shape, dtype=np.complex64):
    return (rng.standard_normal(shape) + 1j * rng.standard_normal(shape)).astype(dtype)


def odot(a, b):
    """Real inner product: sum re*re + im*im."""
    return float(np.sum(a.real * b.real + a.imag * b.imag))


def triples(lx, ly, maxl=-1):
    out = []
    for l1 in sorted(lx):
        for l2 in sorted(ly):
            for l in range(abs(l1 - l2), l1 + l2 + 1):
                if maxl < 0 or l <= maxl:
                    out.append((l1, l2, l))
    return out
