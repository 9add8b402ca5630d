"""ctypes binding of ``libgelib_hip.so`` (the C ABI declared in ``include/gelib_hip.h``).

Tensors are ``torch.complex64`` on the GPU with shape ``(batch, [grid...], 2l+1, channels)``; they are
passed as 5-D descriptors of pointer, dims and strides.  Every call is queued on torch's current HIP
stream.  A missing library or a non-zero status raises; nothing here falls back to another implementation.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libgelib_hip.so")

SYMBOLS = [
    "gelib_hip_strerror", "gelib_hip_last_runtime_error", "gelib_hip_version", "gelib_hip_cg_matrix",
    "gelib_hip_so3type_product",
    "gelib_hip_so3part_cg_fwd", "gelib_hip_so3part_cg_back0", "gelib_hip_so3part_cg_back1",
    "gelib_hip_so3part_diagcg_fwd", "gelib_hip_so3part_diagcg_back0", "gelib_hip_so3part_diagcg_back1",
    "gelib_hip_so3vec_cg_fwd", "gelib_hip_so3vec_cg_bwd", "gelib_hip_so3vec_diagcg_fwd",
    "gelib_hip_so3vec_diagcg_bwd", "gelib_hip_so3part_spharm", "gelib_hip_gather_map_create",
    "gelib_hip_gather_map_destroy", "gelib_hip_part_gather", "gelib_hip_part_mix_channels",
    "gelib_hip_part_mix_channels_static", "gelib_hip_part_mix_channels_wgrad", "gelib_hip_part_mix_workspace_bytes",
    "gelib_hip_so3vec_cg_linear_fwd", "gelib_hip_so3vec_cg_linear_workspace_bytes",
    "gelib_hip_so3vec_cg_linear_bwd", "gelib_hip_so3vec_cg_linear_bwd_workspace_bytes",
    "gelib_hip_set_option", "gelib_hip_set_stream_workspace",
    "gelib_hip_last_path",
    "gelib_hip_malloc", "gelib_hip_free", "gelib_hip_memcpy", "gelib_hip_memset", "gelib_hip_synchronize",
]


class PartDesc(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("dims", ctypes.c_int64 * 5), ("strides", ctypes.c_int64 * 5)]


class GelibHipError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("GElib error: %s (status %d)" % (message, status))
        self.status = status


_lib = None


def lib():
    """Load the library; raises OSError with the build hint if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise OSError("%s is missing: build it with `make -C gelib_amd/csrc` "
                          "(or `python -c 'import __graft_entry__ as g; g.build()'`)" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        P = ctypes.POINTER(PartDesc)
        for name in ("gelib_hip_strerror", "gelib_hip_last_runtime_error", "gelib_hip_version"):
            getattr(L, name).restype = ctypes.c_char_p
        L.gelib_hip_strerror.argtypes = [ctypes.c_int]
        L.gelib_hip_cg_matrix.argtypes = [ctypes.c_int] * 3 + [ctypes.c_void_p]
        L.gelib_hip_so3type_product.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_int),
                                                ctypes.POINTER(ctypes.c_int), ctypes.c_int,
                                                ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int),
                                                ctypes.c_int, ctypes.POINTER(ctypes.c_int64), ctypes.c_int]
        for name in SYMBOLS[5:11]:
            getattr(L, name).argtypes = [P, P, P, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
        for name in ("gelib_hip_so3vec_cg_fwd", "gelib_hip_so3vec_diagcg_fwd"):
            getattr(L, name).argtypes = [ctypes.c_int, P, ctypes.c_int, P, ctypes.c_int, P, ctypes.c_int,
                                         ctypes.c_void_p]
        for name in ("gelib_hip_so3vec_cg_bwd", "gelib_hip_so3vec_diagcg_bwd"):
            getattr(L, name).argtypes = [P, P, ctypes.c_int, P, ctypes.c_int, P, ctypes.c_int, P, ctypes.c_int,
                                         ctypes.c_void_p]
        L.gelib_hip_so3part_spharm.argtypes = [P, ctypes.c_void_p, ctypes.POINTER(ctypes.c_int64),
                                               ctypes.POINTER(ctypes.c_int64), ctypes.c_int, ctypes.c_void_p]
        I32 = ctypes.POINTER(ctypes.c_int32)
        L.gelib_hip_gather_map_create.argtypes = [I32, I32, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                                  ctypes.POINTER(ctypes.c_void_p)]
        L.gelib_hip_gather_map_destroy.argtypes = [ctypes.c_void_p]
        L.gelib_hip_part_gather.argtypes = [P, P, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                            ctypes.c_void_p]
        L.gelib_hip_part_mix_channels.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64,
                                                  ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int64,
                                                  ctypes.c_int, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p]
        L.gelib_hip_part_mix_channels_wgrad.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                                        ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int64,
                                                        ctypes.c_int64, ctypes.c_void_p, ctypes.c_uint64,
                                                        ctypes.c_void_p]
        L.gelib_hip_part_mix_channels_static.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                                         ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int64,
                                                         ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]
        L.gelib_hip_so3vec_cg_linear_fwd.argtypes = [ctypes.c_int, P, ctypes.c_int, P, ctypes.c_int, P,
                                                     ctypes.POINTER(ctypes.c_void_p), ctypes.c_int, ctypes.c_void_p,
                                                     ctypes.c_uint64, ctypes.c_void_p]
        L.gelib_hip_so3vec_cg_linear_bwd.argtypes = [P, P, ctypes.c_void_p, ctypes.c_int, P, ctypes.c_int, P, ctypes.c_int, P,
                                                     ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_uint64,
                                                     ctypes.c_void_p]
        L.gelib_hip_so3vec_cg_linear_bwd_workspace_bytes.restype = ctypes.c_uint64
        L.gelib_hip_so3vec_cg_linear_bwd_workspace_bytes.argtypes = [ctypes.c_int, P, ctypes.c_int, P, ctypes.c_int, P,
                                                                     ctypes.c_int64]
        L.gelib_hip_so3vec_cg_linear_workspace_bytes.restype = ctypes.c_uint64
        L.gelib_hip_so3vec_cg_linear_workspace_bytes.argtypes = [ctypes.c_int, P, ctypes.c_int, P, ctypes.c_int, P]
        L.gelib_hip_part_mix_workspace_bytes.restype = ctypes.c_uint64
        L.gelib_hip_part_mix_workspace_bytes.argtypes = [ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int]
        L.gelib_hip_set_option.argtypes = [ctypes.c_char_p, ctypes.c_int]
        L.gelib_hip_set_stream_workspace.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64]
        _lib = L
    return _lib


def check(status):
    if status != 0:
        L = lib()
        msg = L.gelib_hip_strerror(status).decode()
        if status == 10:
            msg += ": " + L.gelib_hip_last_runtime_error().decode()
        raise GelibHipError(status, msg)


def desc(t):
    """5-D descriptor of a complex64 tensor shaped (b, [g0, [g1]], 2l+1, n)."""
    import torch
    if t.dtype != torch.complex64:
        raise TypeError("SO3parts are complex64 tensors")
    if t.dim() < 3 or t.dim() > 5:
        raise ValueError("an SO3part view has 3 to 5 dimensions (batch, [grid], 2l+1, channels)")
    d = PartDesc()
    d.ptr = t.data_ptr() if t.numel() > 0 else None
    shape = list(t.shape)
    strides = list(t.stride())
    k = t.dim() - 3
    dims = [shape[0]] + shape[1:1 + k] + [1] * (2 - k) + shape[-2:]
    strs = [strides[0]] + strides[1:1 + k] + [0] * (2 - k) + strides[-2:]
    for i in range(5):
        d.dims[i] = dims[i]
        d.strides[i] = strs[i]
    return d


def _stream(t):
    import torch
    dev = t.device if t.is_cuda else None      # a host tensor is refused by the library itself (status 8)
    return ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)


def _arr(tensors):
    if tensors is None:
        return None
    return (PartDesc * len(tensors))(*[desc(t) for t in tensors])


def cg_matrix(l1, l2, l):
    import numpy as np
    out = np.zeros((2 * l1 + 1, 2 * l2 + 1), dtype=np.float32)
    check(lib().gelib_hip_cg_matrix(l1, l2, l, out.ctypes.data))
    return out


def so3type_product(taux, tauy, maxl=-1, diag=False):
    lx, ly = sorted(taux), sorted(tauy)
    n = (max(lx) + max(ly) + 1) if lx and ly else 0
    out = (ctypes.c_int64 * max(n, 1))()
    I = ctypes.c_int
    rc = lib().gelib_hip_so3type_product(int(diag), len(lx), (I * len(lx))(*lx), (I * len(lx))(*[taux[l] for l in lx]),
                                         len(ly), (I * len(ly))(*ly), (I * len(ly))(*[tauy[l] for l in ly]), maxl, out, n)
    if rc < 0:
        check(-rc)
    return {l: int(out[l]) for l in range(n) if out[l] > 0}


def _part(name, dst, a, b, offs, accumulate):
    check(getattr(lib(), name)(ctypes.byref(desc(dst)), ctypes.byref(desc(a)), ctypes.byref(desc(b)), int(offs),
                               int(accumulate), _stream(dst)))


def so3part_cg_fwd(r, x, y, offs=0, accumulate=True):
    _part("gelib_hip_so3part_cg_fwd", r, x, y, offs, accumulate)


def so3part_cg_back0(xg, g, y, offs=0, accumulate=True):
    _part("gelib_hip_so3part_cg_back0", xg, g, y, offs, accumulate)


def so3part_cg_back1(yg, g, x, offs=0, accumulate=True):
    _part("gelib_hip_so3part_cg_back1", yg, g, x, offs, accumulate)


def so3part_diagcg_fwd(r, x, y, offs=0, accumulate=True):
    _part("gelib_hip_so3part_diagcg_fwd", r, x, y, offs, accumulate)


def so3part_diagcg_back0(xg, g, y, offs=0, accumulate=True):
    _part("gelib_hip_so3part_diagcg_back0", xg, g, y, offs, accumulate)


def so3part_diagcg_back1(yg, g, x, offs=0, accumulate=True):
    _part("gelib_hip_so3part_diagcg_back1", yg, g, x, offs, accumulate)


def so3vec_fwd(rparts, xparts, yparts, accumulate=True, diag=False):
    fn = lib().gelib_hip_so3vec_diagcg_fwd if diag else lib().gelib_hip_so3vec_cg_fwd
    check(fn(len(rparts), _arr(rparts), len(xparts), _arr(xparts), len(yparts), _arr(yparts), int(accumulate),
             _stream(rparts[0])))


def so3vec_bwd(xgparts, ygparts, gparts, xparts, yparts, accumulate=True, diag=False):
    """Either gradient list may be None to skip it (back0-only / back1-only)."""
    fn = lib().gelib_hip_so3vec_diagcg_bwd if diag else lib().gelib_hip_so3vec_cg_bwd
    check(fn(_arr(xgparts), _arr(ygparts), len(gparts), _arr(gparts), len(xparts), _arr(xparts), len(yparts),
             _arr(yparts), int(accumulate), _stream(gparts[0])))


UNSUPPORTED = 15


def so3vec_cg_linear_fwd(rparts, xparts, yparts, wparts, accumulate=False):
    """rparts[k] (+)= CGproduct(x, y)[l of rparts[k]] @ wparts[k] in one pass that never stores the product.  False
    (nothing launched) when the shapes are not ones the fused kernel takes; every other failure raises."""
    import torch
    L = lib()
    ra, xa, ya = _arr(rparts), _arr(xparts), _arr(yparts)
    nbytes = int(L.gelib_hip_so3vec_cg_linear_workspace_bytes(len(rparts), ra, len(xparts), xa, len(yparts), ya))
    if nbytes == 0:
        return False
    ws = torch.empty(nbytes, dtype=torch.uint8, device=rparts[0].device)
    wp = (ctypes.c_void_p * len(wparts))(*[w.data_ptr() for w in wparts])
    rc = L.gelib_hip_so3vec_cg_linear_fwd(len(rparts), ra, len(xparts), xa, len(yparts), ya, wp, int(accumulate),
                                          ctypes.c_void_p(ws.data_ptr()), nbytes, _stream(rparts[0]))
    if rc == UNSUPPORTED:
        return False
    check(rc)
    return True


def so3vec_cg_linear_bwd(xgparts, ygparts, wgparts, gparts, xparts, yparts, wparts, accumulate=False,
                         workspace_bytes=1 << 30):
    """Gradients of CGproduct(x, y) @ W with respect to x, y and the matrices (any of the three lists may be None), given
    the gradient gparts of the result, in the memory of one chunk of the batch: the product and its gradient exist only
    for the chunk at hand, in a workspace of at most workspace_bytes (more when one batch entry needs more).  False
    (nothing launched) when the shapes are not ones the call takes."""
    import torch
    L = lib()
    ga, xa, ya = _arr(gparts), _arr(xparts), _arr(yparts)
    args = (len(gparts), ga, len(xparts), xa, len(yparts), ya)
    whole = int(L.gelib_hip_so3vec_cg_linear_bwd_workspace_bytes(*args, 0))
    if whole == 0:
        return False
    one = int(L.gelib_hip_so3vec_cg_linear_bwd_workspace_bytes(*args, 1))
    nbytes = whole if whole <= workspace_bytes else max(one, workspace_bytes)
    ws = torch.empty(nbytes + 256, dtype=torch.uint8, device=gparts[0].device)
    base = (ws.data_ptr() + 255) & ~255
    wp = (ctypes.c_void_p * len(wparts))(*[w.data_ptr() for w in wparts])
    wgp = (ctypes.c_void_p * len(wgparts))(*[w.data_ptr() for w in wgparts]) if wgparts is not None else None
    rc = L.gelib_hip_so3vec_cg_linear_bwd(_arr(xgparts), _arr(ygparts), wgp, len(gparts), ga, len(xparts), xa, len(yparts),
                                          ya, wp, int(accumulate), ctypes.c_void_p(base), nbytes, _stream(gparts[0]))
    if rc == UNSUPPORTED:
        return False
    check(rc)
    return True


def set_stream_workspace(buf, stream=None):
    """Lends the library the uint8 tensor buf (None: takes the loan back) as its scratch on `stream` (torch's current
    stream of buf's device by default).  The caller keeps buf alive while calls or graphs may use it."""
    import torch
    if stream is None:
        stream = torch.cuda.current_stream(buf.device if buf is not None else None)
    sp = ctypes.c_void_p(stream.cuda_stream)
    if buf is None:
        check(lib().gelib_hip_set_stream_workspace(sp, None, 0))
        return
    base = (buf.data_ptr() + 255) & ~255
    check(lib().gelib_hip_set_stream_workspace(sp, ctypes.c_void_p(base), buf.numel() - (base - buf.data_ptr())))


def so3part_spharm(r, x, accumulate=True):
    """r (b, [grid], 2l+1, n) complex64 (+)= spherical harmonics of the float32 vectors x (b or 1, [grid], 3, n)."""
    import torch
    if x.dtype != torch.float32:
        raise TypeError("the vectors are float32")
    if x.dim() != r.dim() or x.size(-2) != 3:
        raise ValueError("x is shaped like r with 3 in place of 2l+1")
    k = x.dim() - 3
    dims = [x.shape[0]] + list(x.shape[1:1 + k]) + [1] * (2 - k) + list(x.shape[-2:])
    strs = [x.stride(0)] + list(x.stride()[1:1 + k]) + [0] * (2 - k) + list(x.stride()[-2:])
    A = ctypes.c_int64 * 5
    check(lib().gelib_hip_so3part_spharm(ctypes.byref(desc(r)), ctypes.c_void_p(x.data_ptr()), A(*dims), A(*strs),
                                         int(accumulate), _stream(r)))


class GatherMap:
    """Device form of a list of (source, target) pairs; freed with the object."""

    def __init__(self, sources, targets, n_in, n_out):
        n = len(sources)
        if len(targets) != n:
            raise ValueError("as many sources as targets are needed")
        A = ctypes.c_int32 * max(n, 1)
        self.handle = ctypes.c_void_p()
        self.n_in, self.n_out = n_in, n_out
        check(lib().gelib_hip_gather_map_create(A(*sources), A(*targets), n, n_in, n_out, ctypes.byref(self.handle)))

    def __del__(self):
        if getattr(self, "handle", None):
            lib().gelib_hip_gather_map_destroy(self.handle)
            self.handle = None


def part_gather(r, x, gmap, dim, inverse=False, accumulate=True):
    """r[.., t, ..] (+)= sum over the pairs (s, t) of x[.., s, ..] along dimension dim (0 = batch, 1..2 = grid) of the
    5-D views; inverse swaps the roles of sources and targets."""
    check(lib().gelib_hip_part_gather(ctypes.byref(desc(r)), ctypes.byref(desc(x)), gmap.handle, int(dim), int(inverse),
                                      int(accumulate), _stream(r)))


def mix_channels_ok(x):
    """True if part_mix_channels takes x as it is: contiguous rows of an even number of channels, 16-byte aligned."""
    return x.is_contiguous() and x.shape[-1] > 0 and x.shape[-1] % 2 == 0 and x.data_ptr() % 16 == 0


def mix_workspace(kind, rows, n_in, n_out, device):
    """The workspace a channel-mixing call needs (kind 0: part_mix_channels, 1: part_mix_channels_wgrad), taken from
    torch's caching allocator: it is stream-ordered, so the buffer is not handed to anybody else before the kernels
    queued on the current stream have read it, and the library itself never allocates."""
    import torch
    nbytes = int(lib().gelib_hip_part_mix_workspace_bytes(kind, rows, n_in, n_out))
    return torch.empty(max(nbytes, 16), dtype=torch.uint8, device=device), nbytes


def part_mix_channels(r, x, w, adjoint=False):
    """r[..., o] = sum_c x[..., c] V[c, o] with V = w (n_in, n_out), or V = w^H for w (n_out, n_in) when adjoint.
    r and x are contiguous complex64 tensors that differ only in their last extent."""
    n_in, n_out = x.shape[-1], r.shape[-1]
    if tuple(w.shape) != ((n_out, n_in) if adjoint else (n_in, n_out)) or r.shape[:-1] != x.shape[:-1]:
        raise ValueError("shapes of r, x and w do not fit")
    if not (r.is_contiguous() and x.is_contiguous() and w.is_contiguous()):
        raise ValueError("contiguous tensors are needed")
    rows = x.numel() // n_in if n_in else 0
    ws, nbytes = mix_workspace(0, rows, n_in, n_out, r.device)
    check(lib().gelib_hip_part_mix_channels(r.data_ptr(), x.data_ptr(), w.data_ptr(), rows, n_in, n_out, n_out, n_in,
                                            int(adjoint), ws.data_ptr(), nbytes, _stream(r)))


def part_mix_channels_wgrad(wg, x, g):
    """wg (n_in, n_out) = sum over the leading indices of conj(x[..., c]) g[..., o] for contiguous complex64 tensors."""
    n_in, n_out = x.shape[-1], g.shape[-1]
    if tuple(wg.shape) != (n_in, n_out) or g.shape[:-1] != x.shape[:-1]:
        raise ValueError("shapes of wg, x and g do not fit")
    if not (wg.is_contiguous() and x.is_contiguous() and g.is_contiguous()):
        raise ValueError("contiguous tensors are needed")
    rows = x.numel() // n_in if n_in else 0
    ws, nbytes = mix_workspace(1, rows, n_in, n_out, wg.device)
    check(lib().gelib_hip_part_mix_channels_wgrad(wg.data_ptr(), x.data_ptr(), g.data_ptr(), rows, n_in, n_out, n_in,
                                                  n_out, ws.data_ptr(), nbytes, _stream(wg)))


def set_option(name, value):
    check(lib().gelib_hip_set_option(name.encode(), int(value)))


def last_path():
    return lib().gelib_hip_last_path()
