"""The C++ mirror of GElib's interface (include/gelib/GElib.hpp): the demo program builds parts and vecs on the GPU
with the reference's constructor / CGproduct / Gpart_add_* calls; its dumped results are checked against the CPU
oracle here."""
import os
import struct
import subprocess

import numpy as np
import pytest

from oracle import cg_oracle as ora
from tests import gpu_util as U

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
DEMO = os.path.join(HERE, "cpp", "so3_api_demo")


def read_tensors(path):
    out = []
    with open(path, "rb") as f:
        data = f.read()
    pos = 0
    while pos < len(data):
        (nd,) = struct.unpack_from("i", data, pos)
        pos += 4
        dims = struct.unpack_from("%di" % nd, data, pos)
        pos += 4 * nd
        n = int(np.prod(dims))
        out.append(np.frombuffer(data, dtype=np.complex64, count=n, offset=pos).reshape(dims).copy())
        pos += 8 * n
    return out


def test_cpp_api_demo(tmp_path):
    assert os.path.exists(DEMO), "build it with `make -C tests/cpp` (done by __graft_entry__.build())"
    out = tmp_path / "demo.bin"
    res = subprocess.run([DEMO, str(out)], capture_output=True, text=True, timeout=100)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "so3_api_demo ok" in res.stdout
    t = read_tensors(str(out))
    x, y, r, g, xg, yg = t[:6]
    assert r.shape == (3, 5, 32)
    assert U.gate_excess(r, ora.cg_fwd(x, y, 2)) <= 1.0
    wxg, wyg = ora.cg_bwd(g, x, y)
    c = lambda a: a.astype(np.complex128)
    exg, eyg = ora.cg_bwd(c(g), c(x), c(y))
    U.assert_parity(xg, wxg, exg, ora.part_term_sums(ora.CG_BACK0, g, x, y), "C++ back0")
    U.assert_parity(yg, wyg, eyg, ora.part_term_sums(ora.CG_BACK1, g, x, y), "C++ back1")
    u, v, w = t[6:9], t[9:12], t[12:]
    want = ora.vec_fwd(u, v, 2)
    assert [p.shape for p in w] == [p.shape for p in want]
    for a, b in zip(w, want):
        assert U.gate_excess(a, b) <= 1.0
