"""ctypes front-end of the CPU oracle (``cg_oracle.c``).  TEST INFRASTRUCTURE ONLY.

Only the test-suite, the smoke check and the ``cpu_baseline`` leg of the benchmark import this
module; the shipped package never does.  Arrays are numpy ``complex64`` (loop-order-faithful float32
path) or ``complex128`` (float64 path) of shape ``(B, 2l+1, N)`` with arbitrary strides.

``gather`` is parity unpinned: the loop the reference calls for it (cnine::GatherSlices) is outside its tree.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcg_oracle.so")

CG_FWD, CG_BACK0, CG_BACK1, DIAG_FWD, DIAG_BACK0, DIAG_BACK1 = range(6)


def build(force=False):
    """Compile ``cg_oracle.c`` with gcc (a few seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libcg_oracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


class _Part(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("B", ctypes.c_int64), ("M", ctypes.c_int64), ("N", ctypes.c_int64),
                ("sb", ctypes.c_int64), ("sm", ctypes.c_int64), ("sc", ctypes.c_int64)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        L.ora_cg_coeff.restype = ctypes.c_double
        L.ora_cg_coeff.argtypes = [ctypes.c_int] * 5
        L.ora_cg_matrix.restype = ctypes.c_int
        L.ora_cg_matrix.argtypes = [ctypes.c_int] * 3 + [ctypes.c_void_p]
        L.ora_part_op.restype = ctypes.c_int
        L.ora_part_op.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(_Part), ctypes.POINTER(_Part),
                                  ctypes.POINTER(_Part), ctypes.c_int, ctypes.c_int]
        L.ora_vec_op.restype = ctypes.c_int
        L.ora_vec_op.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.POINTER(_Part), ctypes.c_int,
                                 ctypes.POINTER(_Part), ctypes.c_int, ctypes.POINTER(_Part), ctypes.c_int]
        L.ora_type_product.restype = ctypes.c_int
        L.ora_max_threads.restype = ctypes.c_int
        _lib = L
    return _lib


def max_threads():
    return lib().ora_max_threads()


def cg_coeff(l1, l2, l, m1, m2):
    return lib().ora_cg_coeff(l1, l2, l, m1, m2)


def cg_matrix(l1, l2, l):
    out = np.zeros((2 * l1 + 1, 2 * l2 + 1), dtype=np.float32)
    rc = lib().ora_cg_matrix(l1, l2, l, out.ctypes.data)
    if rc:
        raise ValueError("l outside the triangle")
    return out


def _prec(a):
    if a.dtype == np.complex64:
        return 32
    if a.dtype == np.complex128:
        return 64
    raise TypeError("oracle arrays must be complex64 or complex128")


def _desc(a):
    assert a.ndim == 3, "oracle parts are (B, 2l+1, N)"
    isz = a.itemsize
    assert all(s % isz == 0 for s in a.strides)
    return _Part(a.ctypes.data, a.shape[0], a.shape[1], a.shape[2], a.strides[0] // isz, a.strides[1] // isz,
                 a.strides[2] // isz)


_ERR = {1: "bad op/precision", 2: "even m-dimension", 3: "l outside the triangle", 4: "Diag needs N1==N2",
        5: "offs+n_out exceeds the product's channels", 6: "batch dimensions cannot be reconciled"}


def part_op(op, r, x, y, offs=0, nthreads=1):
    """In-place reference loop nest.  Roles (r, x, y): forward adds into r, back0 into x, back1 into y."""
    p = _prec(r)
    assert _prec(x) == p and _prec(y) == p
    rc = lib().ora_part_op(op, p, ctypes.byref(_desc(r)), ctypes.byref(_desc(x)), ctypes.byref(_desc(y)), offs,
                           nthreads)
    if rc:
        raise ValueError(_ERR.get(rc, str(rc)))


def vec_op(op, rparts, xparts, yparts, nthreads=1):
    """Vec-level loops over every (l1,l2,l) triple; part lists are sorted by l here."""
    xs = sorted(xparts, key=lambda a: a.shape[1])
    ys = sorted(yparts, key=lambda a: a.shape[1])
    rs = sorted(rparts, key=lambda a: a.shape[1])
    p = _prec(xs[0])
    X = (_Part * len(xs))(*[_desc(a) for a in xs])
    Y = (_Part * len(ys))(*[_desc(a) for a in ys])
    R = (_Part * len(rs))(*[_desc(a) for a in rs])
    rc = lib().ora_vec_op(op, p, len(xs), X, len(ys), Y, len(rs), R, nthreads)
    if rc:
        raise ValueError(_ERR.get(rc, str(rc)))


def type_product(taux, tauy, maxl=-1, diag=False):
    """{l: n} x {l: n} -> {l: n_out}: the type of the (Diag)CGproduct."""
    lx = sorted(taux)
    ly = sorted(tauy)
    n = 2 * (max(lx) + max(ly)) + 2
    out = (ctypes.c_int64 * n)()
    LX = (ctypes.c_int * len(lx))(*lx)
    CX = (ctypes.c_int * len(lx))(*[taux[l] for l in lx])
    LY = (ctypes.c_int * len(ly))(*ly)
    CY = (ctypes.c_int * len(ly))(*[tauy[l] for l in ly])
    rc = lib().ora_type_product(int(diag), len(lx), LX, CX, len(ly), LY, CY, maxl, out, n)
    assert rc >= 0
    return {l: int(out[l]) for l in range(n) if out[l] > 0}


# ---- value-returning conveniences ------------------------------------------------------------------------------

def _bmax(*arrs):
    return max(a.shape[0] for a in arrs)


def cg_fwd(x, y, l, diag=False, nthreads=1):
    n = x.shape[2] if diag else x.shape[2] * y.shape[2]
    r = np.zeros((_bmax(x, y), 2 * l + 1, n), dtype=x.dtype)
    part_op(DIAG_FWD if diag else CG_FWD, r, x, y, 0, nthreads)
    return r


def cg_bwd(g, x, y, diag=False, nthreads=1):
    xg = np.zeros_like(x)
    yg = np.zeros_like(y)
    part_op(DIAG_BACK0 if diag else CG_BACK0, g, xg, y, 0, nthreads)
    part_op(DIAG_BACK1 if diag else CG_BACK1, g, x, yg, 0, nthreads)
    return xg, yg


def vec_fwd(xparts, yparts, maxl=-1, diag=False, nthreads=1):
    taux = {(a.shape[1] - 1) // 2: a.shape[2] for a in xparts}
    tauy = {(a.shape[1] - 1) // 2: a.shape[2] for a in yparts}
    tau = type_product(taux, tauy, maxl, diag)
    B = _bmax(xparts[0], yparts[0])
    rparts = [np.zeros((B, 2 * l + 1, n), dtype=xparts[0].dtype) for l, n in sorted(tau.items())]
    vec_op(DIAG_FWD if diag else CG_FWD, rparts, xparts, yparts, nthreads)
    return rparts


def vec_bwd(gparts, xparts, yparts, diag=False, nthreads=1):
    xg = [np.zeros_like(a) for a in xparts]
    yg = [np.zeros_like(a) for a in yparts]
    vec_op(DIAG_BACK0 if diag else CG_BACK0, gparts, xg, yparts, nthreads)
    vec_op(DIAG_BACK1 if diag else CG_BACK1, gparts, xparts, yg, nthreads)
    return xg, yg


def _moduli(parts):
    return [np.abs(a).astype(np.complex128) for a in parts]


def part_term_sums(op, r, x, y, offs=0):
    """Term sums of one part-level operation, for its destination (r forward, x back0, y back1): the float64 loop
    nest with |C| on the moduli of the other two tensors, started from zero.  Arrays as for part_op."""
    parts = [_moduli([a])[0] for a in (r, x, y)]
    dest = parts[0 if op in (CG_FWD, DIAG_FWD) else 1 if op in (CG_BACK0, DIAG_BACK0) else 2]
    dest[...] = 0
    lib().ora_set_abs_coeffs(1)
    try:
        part_op(op, parts[0], parts[1], parts[2], offs)
    finally:
        lib().ora_set_abs_coeffs(0)
    return dest.real.copy()


def vec_fwd_term_sums(xparts, yparts, maxl=-1, diag=False, nthreads=1):
    """For every element of the product, the sum of the moduli of its terms, sum |C| |x| |y| (float64, real).
    Error-analysis aid: the rounding error of a float32 evaluation of an element scales with this sum."""
    lib().ora_set_abs_coeffs(1)
    try:
        return [p.real.copy() for p in vec_fwd(_moduli(xparts), _moduli(yparts), maxl, diag, nthreads)]
    finally:
        lib().ora_set_abs_coeffs(0)


def vec_bwd_term_sums(gparts, xparts, yparts, diag=False, nthreads=1):
    """The same for both gradients: sum |C| |g| |y| per element of xg and sum |C| |g| |x| per element of yg."""
    lib().ora_set_abs_coeffs(1)
    try:
        xg, yg = vec_bwd(_moduli(gparts), _moduli(xparts), _moduli(yparts), diag, nthreads)
        return [p.real.copy() for p in xg], [p.real.copy() for p in yg]
    finally:
        lib().ora_set_abs_coeffs(0)


def cg_term_sums(g, x, y, l, diag=False, nthreads=1):
    """The same for one triple: the sums for the product part l and for the two gradients of g."""
    lib().ora_set_abs_coeffs(1)
    try:
        (mg,), (mx,), (my,) = _moduli([g]), _moduli([x]), _moduli([y])
        r = cg_fwd(mx, my, l, diag, nthreads)
        xg, yg = cg_bwd(mg, mx, my, diag, nthreads)
        return r.real.copy(), xg.real.copy(), yg.real.copy()
    finally:
        lib().ora_set_abs_coeffs(0)


def spharm(l, x, batch=None):
    """(B or 1, 3, n) float32 vectors -> (B, 2l+1, n) complex64 spherical harmonics, the reference's add_spharm into zeros."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert x.ndim == 3 and x.shape[1] == 3
    B = batch or x.shape[0]
    assert x.shape[0] in (1, B)
    r = np.zeros((B, 2 * l + 1, x.shape[2]), dtype=np.complex64)
    f = lib().ora_spharm
    f.restype = ctypes.c_int
    f.argtypes = [ctypes.c_int, ctypes.c_longlong, ctypes.c_longlong, ctypes.c_void_p, ctypes.c_longlong,
                  ctypes.c_longlong, ctypes.c_void_p]
    xsb = 0 if x.shape[0] == 1 else 3 * x.shape[2]   # one set of vectors is shared by the whole batch
    rc = f(l, B, x.shape[2], x.ctypes.data, xsb, x.shape[2], r.ctypes.data)
    assert rc == 0
    return r


def gather(x, sources, targets, n_out, axis, r=None):
    """r[.., t, ..] += x[.., s, ..] for every pair (s, t), pairs taken in the order given within one target: the call
    sites of the reference's gather (core/Gpart.hpp:537-563; the loop itself, cnine::GatherSlices, is not in its
    tree, so this function is unpinned by the reference and pinned only by its definition as a 0/1 matrix product,
    see the tests).  float32 adds in pair order, so the result is reproducible bit for bit."""
    shape = list(x.shape)
    shape[axis] = n_out
    out = np.zeros(shape, dtype=x.dtype) if r is None else r
    xs = np.moveaxis(x, axis, 0)
    os_ = np.moveaxis(out, axis, 0)
    for s, t in zip(sources, targets):
        os_[t] += xs[s]
    return out
