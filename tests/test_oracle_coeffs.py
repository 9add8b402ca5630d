"""Pins the oracle's Clebsch-Gordan coefficients (ora_cg_coeff / ora_cg_matrix) without the reference:
exact sympy radicals, the table printed in the reference's docs, orthogonality and symmetry identities."""
import numpy as np
import pytest

from oracle import cg_oracle as ora
from tests import helpers as H


def test_doc_table_1_2_2():
    # python/docs/source/SO3CG.rst:51-53 prints the (1,2,2) matrix to 4 decimals
    doc = np.array([[0, -0.5774, -0.7071, -0.7071, -0.5774],
                    [0.8165, 0.4082, 0, -0.4082, -0.8165],
                    [0.5774, 0.7071, 0.7071, 0.5774, 0]])
    C = ora.cg_matrix(1, 2, 2)
    assert C.shape == (3, 5) and C.dtype == np.float32
    assert np.max(np.abs(C - doc)) < 6e-5


def test_against_sympy_fixture():
    tabs = H.golden_cg_tables()
    assert len(tabs) >= 85
    worst = 0.0
    for (l1, l2, l), T in tabs.items():
        C = ora.cg_matrix(l1, l2, l)
        assert C.shape == T.shape
        # stored as float: compare against the float-rounded exact value, allow one ulp
        err = np.max(np.abs(C.astype(np.float64) - T))
        assert err <= 1.2e-7 * max(1.0, np.max(np.abs(T))), (l1, l2, l, err)
        for m1 in range(-l1, l1 + 1):
            for m2 in range(-l2, l2 + 1):
                if abs(m1 + m2) <= l:
                    d = abs(ora.cg_coeff(l1, l2, l, m1, m2) - T[m1 + l1, m2 + l2])
                    worst = max(worst, d)
    assert worst < 5e-13, worst


@pytest.mark.parametrize("l1,l2,l", [(3, 2, 4), (2, 2, 0), (5, 3, 7)])
def test_against_live_sympy(l1, l2, l):
    T = H.sympy_cg_matrix(l1, l2, l)
    for m1 in range(-l1, l1 + 1):
        for m2 in range(-l2, l2 + 1):
            if abs(m1 + m2) <= l:
                assert abs(ora.cg_coeff(l1, l2, l, m1, m2) - T[m1 + l1, m2 + l2]) < 1e-13


@pytest.mark.parametrize("l1,l2", [(0, 0), (1, 1), (2, 3), (4, 4), (7, 5), (10, 10)])
def test_orthonormality(l1, l2):
    # sum_{m1,m2} C^l(m1,m2) C^l'(m1,m2) delta_{m,m'} = delta_{l l'}; sum_l C^l(m1,m2)^2 = 1
    ls = list(range(abs(l1 - l2), l1 + l2 + 1))
    W = {l: H.dense_cg_tensor(np.array([[ora.cg_coeff(l1, l2, l, m1, m2) if abs(m1 + m2) <= l else 0.0
                                         for m2 in range(-l2, l2 + 1)] for m1 in range(-l1, l1 + 1)]), l1, l2, l)
         for l in ls}
    for la in ls:
        for lb in ls:
            G = np.einsum("ijm,ijn->mn", W[la], W[lb][:, :, :]) if la == lb else None
            if la == lb:
                assert np.allclose(G, np.eye(2 * la + 1), atol=1e-11)
            else:
                # different l: overlap at equal m must vanish
                for m in range(-min(la, lb), min(la, lb) + 1):
                    ov = np.sum(W[la][:, :, m + la] * W[lb][:, :, m + lb])
                    assert abs(ov) < 1e-11
    tot = sum(np.sum(W[l] ** 2, axis=2) for l in ls)
    assert np.allclose(tot, 1.0, atol=1e-11)


@pytest.mark.parametrize("l1,l2,l", [(1, 2, 2), (2, 3, 4), (4, 4, 3), (6, 5, 2)])
def test_exchange_symmetry(l1, l2, l):
    # <l2 m2; l1 m1 | l m> = (-1)^(l1+l2-l) <l1 m1; l2 m2 | l m>   (SO3/SO3group.hpp:49-51)
    s = 1 - 2 * ((l1 + l2 - l) % 2)
    A = ora.cg_matrix(l1, l2, l)
    Bm = ora.cg_matrix(l2, l1, l)
    assert np.allclose(Bm.T, s * A, atol=1e-7)


def test_special_values():
    # l1=0: C == 1 ; l=l1+l2 stretched state: C(l1,l2)=1 ; l=0: (-1)^(l1-m)/sqrt(2l1+1)
    for l2 in range(5):
        assert np.allclose(ora.cg_matrix(0, l2, l2), 1.0)
    assert abs(ora.cg_coeff(3, 4, 7, 3, 4) - 1.0) < 1e-14
    assert abs(ora.cg_coeff(3, 4, 7, -3, -4) - 1.0) < 1e-14
    for l1 in range(6):
        for m in range(-l1, l1 + 1):
            want = (-1) ** (l1 - m) / np.sqrt(2 * l1 + 1)
            assert abs(ora.cg_coeff(l1, l1, 0, m, -m) - want) < 1e-14


def test_invalid_triangle():
    with pytest.raises(ValueError):
        ora.cg_matrix(1, 1, 3)
