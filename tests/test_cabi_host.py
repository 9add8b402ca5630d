"""CPU-side checks of the C ABI: the library loads, exports every symbol the header declares, its host-side
coefficient bank and type arithmetic agree with the oracle, and every shape error is reported as a status code
before any GPU work is attempted.  No kernel is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest

from gelib_amd import cabi
from oracle import cg_oracle as ora

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "gelib_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gelib_hip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = cabi.lib()
    names = declared_symbols()
    assert len(names) >= 17
    for n in names:
        assert hasattr(L, n), n
    assert sorted(cabi.SYMBOLS) == names
    assert b"gfx950" in L.gelib_hip_version()


def test_bank_matches_oracle():
    for l1 in range(0, 7):
        for l2 in range(0, 7):
            for l in range(abs(l1 - l2), l1 + l2 + 1):
                assert np.array_equal(cabi.cg_matrix(l1, l2, l), ora.cg_matrix(l1, l2, l)), (l1, l2, l)
    for t in [(10, 10, 0), (10, 10, 7), (10, 10, 20), (20, 12, 9), (32, 32, 64)]:
        assert np.array_equal(cabi.cg_matrix(*t), ora.cg_matrix(*t)), t
    with pytest.raises(cabi.GelibHipError) as e:
        cabi.cg_matrix(1, 1, 3)
    assert e.value.status == 3


def test_type_product_known_answers():
    # python/docs/source/abandoned/SO3type.rst:28-41
    assert cabi.so3type_product({0: 2, 1: 2}, {0: 2, 1: 2}) == {0: 8, 1: 12, 2: 4}
    assert cabi.so3type_product({0: 1, 1: 1, 2: 1}, {0: 1, 1: 1, 2: 1}) == {0: 3, 1: 6, 2: 6, 3: 3, 4: 1}
    assert cabi.so3type_product({0: 1, 1: 1, 2: 1}, {0: 1, 1: 1, 2: 1}, maxl=2) == {0: 3, 1: 6, 2: 6}
    tau = {l: 16 for l in range(5)}
    assert cabi.so3type_product(tau, tau, 4) == ora.type_product(tau, tau, 4)
    assert cabi.so3type_product(tau, tau, -1, diag=True) == ora.type_product(tau, tau, -1, diag=True)


def fake(b, m, n, g=(1, 1), ptr=0x1000):
    d = cabi.PartDesc()
    d.ptr = ptr
    dims = [b, g[0], g[1], m, n]
    st = [g[0] * g[1] * m * n, g[1] * m * n, m * n, n, 1]
    for i in range(5):
        d.dims[i] = dims[i]
        d.strides[i] = st[i]
    return d


def call(name, r, x, y, offs=0):
    fn = getattr(cabi.lib(), name)
    return fn(ctypes.byref(r), ctypes.byref(x), ctypes.byref(y), offs, 1, None)


@pytest.mark.parametrize("name", ["gelib_hip_so3part_cg_fwd", "gelib_hip_so3part_diagcg_fwd"])
def test_shape_errors_are_status_codes(name):
    diag = "diag" in name
    n_out = 4 if diag else 16
    x, y = fake(2, 3, 4), fake(2, 3, 4)
    assert call(name, fake(2, 4, n_out), x, y) == 2            # even m-dimension
    assert call(name, fake(2, 9, n_out), x, y) == 3            # l=4 outside 1 x 1
    assert call(name, fake(2, 3, n_out - 1), x, y) == 5        # not enough channels
    assert call(name, fake(2, 3, n_out), x, y, offs=1) == 5    # offset pushes the block out
    assert call(name, fake(2, 3, n_out), x, y, offs=-1) == 12
    assert call(name, fake(3, 3, n_out), x, y) == 6            # batch 3 vs 2
    assert call(name, fake(2, 3, n_out, g=(2, 2)), fake(2, 3, 4, g=(3, 2)), y) == 7
    assert call(name, fake(2, 3, n_out, ptr=None), x, y) == 1
    fn = getattr(cabi.lib(), name)
    assert fn(None, ctypes.byref(x), ctypes.byref(y), 0, 1, None) == 1
    if diag:
        assert call(name, fake(2, 3, 4), x, fake(2, 3, 5)) == 4


def test_backward_roles():
    # back0(xg, g, y): destination first, gradient second, partner third (core/CGproduct.hpp:65-83)
    g, xg, y = fake(2, 9, 6), fake(2, 5, 2), fake(2, 7, 3)
    assert call("gelib_hip_so3part_cg_back0", xg, g, y, offs=1) == 5
    assert call("gelib_hip_so3part_cg_back0", fake(2, 1, 2), g, fake(2, 3, 3)) == 3   # l=4 outside 0 x 1
    yg, x = fake(2, 7, 3), fake(2, 5, 2)
    assert call("gelib_hip_so3part_cg_back1", yg, g, x, offs=1) == 5


def test_vec_errors():
    L = cabi.lib()
    A = cabi.PartDesc * 2
    x = A(fake(2, 1, 2), fake(2, 3, 2))
    y = A(fake(2, 1, 2), fake(2, 3, 2))
    r_ok = (cabi.PartDesc * 3)(fake(2, 1, 8), fake(2, 3, 12), fake(2, 5, 4))
    r_small = (cabi.PartDesc * 3)(fake(2, 1, 8), fake(2, 3, 11), fake(2, 5, 4))
    assert L.gelib_hip_so3vec_cg_fwd(3, r_small, 2, x, 2, y, 1, None) == 5
    dup = A(fake(2, 3, 2), fake(2, 3, 2))
    assert L.gelib_hip_so3vec_cg_fwd(3, r_ok, 2, dup, 2, y, 1, None) == 9
    ybad = A(fake(3, 1, 2), fake(3, 3, 2))
    assert L.gelib_hip_so3vec_cg_fwd(3, r_ok, 2, x, 2, ybad, 1, None) == 6
    ydiag = A(fake(2, 1, 3), fake(2, 3, 3))
    assert L.gelib_hip_so3vec_diagcg_fwd(3, r_ok, 2, x, 2, ydiag, 1, None) == 4
    # gradient lists must mirror their operands
    xg_bad = A(fake(2, 1, 2), fake(2, 3, 3))
    assert L.gelib_hip_so3vec_cg_bwd(xg_bad, None, 3, r_ok, 2, x, 2, y, 1, None) == 9


def test_host_pointer_is_refused_not_launched():
    # a well-formed call on host memory must come back as a status, never reach a kernel
    buf = np.zeros(2 * 3 * 16, dtype=np.complex64)
    r = fake(2, 3, 16, ptr=buf.ctypes.data)
    x = fake(2, 3, 4, ptr=buf.ctypes.data)
    y = fake(2, 3, 4, ptr=buf.ctypes.data)
    assert call("gelib_hip_so3part_cg_fwd", r, x, y) in (8, 10)


def test_unknown_option():
    assert cabi.lib().gelib_hip_set_option(b"no_such_option", 1) != 0
    cabi.set_option("force_generic", 0)


def test_destination_that_repeats_memory_and_negative_strides():
    """An expanded view as destination (extent > 1, stride 0) and negative strides are refused before any pointer is
    looked at, whatever the "check_pointers" option says."""
    cabi.set_option("check_pointers", 0)
    try:
        x, y = fake(2, 3, 4), fake(2, 3, 4)
        r = fake(2, 3, 16)
        r.strides[0] = 0                                   # the two cells of the product share their memory
        assert call("gelib_hip_so3part_cg_fwd", r, x, y) == 11
        xg, g = fake(2, 3, 4), fake(2, 3, 16)
        xg.strides[4] = 0                                  # all channels of the gradient in one place
        assert call("gelib_hip_so3part_cg_back0", xg, g, y) == 11
        yg = fake(2, 3, 4)
        yg.strides[3] = 0
        assert call("gelib_hip_so3part_cg_back1", yg, g, x) == 11
        neg = fake(2, 3, 4)
        neg.strides[3] = -4
        assert call("gelib_hip_so3part_cg_fwd", fake(2, 3, 16), neg, y) == 12
        L = cabi.lib()
        A = cabi.PartDesc * 1
        rr = A(fake(2, 3, 16))
        rr[0].strides[0] = 0
        assert L.gelib_hip_so3vec_cg_fwd(1, rr, 1, A(x), 1, A(y), 1, None) == 11
        gg = A(fake(2, 3, 16))
        bad = A(fake(2, 3, 4))
        bad[0].strides[0] = 0
        assert L.gelib_hip_so3vec_cg_bwd(bad, None, 1, gg, 1, A(x), 1, A(y), 1, None) == 11
    finally:
        cabi.set_option("check_pointers", 1)


def test_part_count_limits():
    """An SO3vec may hold every l from 0 to 32 (33 parts), its product every l up to 64 (65 parts); one more is status 9."""
    L = cabi.lib()
    xs = (cabi.PartDesc * 34)(*[fake(1, 2 * min(l, 32) + 1, 1) for l in range(34)])   # the last l is a repeat
    y = (cabi.PartDesc * 1)(fake(1, 1, 1))
    r = (cabi.PartDesc * 1)(fake(1, 1, 1))
    assert L.gelib_hip_so3vec_cg_fwd(1, r, 34, xs, 1, y, 1, None) == 9
    # 33 distinct parts pass the part-count check and are stopped later, by the missing channels of r
    assert L.gelib_hip_so3vec_cg_fwd(1, (cabi.PartDesc * 1)(fake(1, 1, 0, ptr=None)), 33, xs, 1, y, 1, None) in (0, 5)
    assert L.gelib_hip_part_mix_workspace_bytes(0, 10, 32, 16) >= 16 * 32 * 16
    assert L.gelib_hip_part_mix_workspace_bytes(2, 10, 32, 16) == 0
