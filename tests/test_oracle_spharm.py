"""The spherical-harmonics restatement of the oracle (SO3/SO3part.hpp:340-403) pinned without the reference:
scipy's spherical harmonics (the reference's own check, python/tests/test_spharm.py), the printed example of the
reference's documentation, the polar-axis special case and closed forms for l = 0, 1."""
import numpy as np
import pytest

from oracle import cg_oracle as ora

scipy_special = pytest.importorskip("scipy.special")


def scipy_ylm(l, X):
    nm = np.linalg.norm(X.astype(np.float64), axis=1)
    theta = np.arccos(X[:, 2, :] / nm)
    phi = np.arctan2(X[:, 1, :].astype(np.float64), X[:, 0, :].astype(np.float64))
    if hasattr(scipy_special, "sph_harm_y"):
        return np.stack([scipy_special.sph_harm_y(l, m, theta, phi) for m in range(-l, l + 1)], axis=1)
    return np.stack([scipy_special.sph_harm(m, l, phi, theta) for m in range(-l, l + 1)], axis=1)


@pytest.mark.parametrize("l", [0, 1, 2, 4, 7, 10, 20])
def test_against_scipy(l):
    X = np.random.default_rng(l).standard_normal((4, 3, 6)).astype(np.float32)
    got = ora.spharm(l, X)
    want = scipy_ylm(l, X)
    assert got.shape == (4, 2 * l + 1, 6)
    assert np.max(np.abs(got - want)) <= 2e-5 * max(1.0, np.max(np.abs(want)))   # float32 recurrences


def test_documented_example():
    # python/docs/source/abandoned/SO3part.rst:170-176: gelib.SO3part.spharm(2,[0.12,0.31,-0.55])
    got = ora.spharm(2, np.array([[[0.12], [0.31], [-0.55]]], dtype=np.float32))[0, :, 0]
    want = np.array([-0.0764131 - 0.0695855j, -0.123458 + 0.318933j, 0.37763, 0.123458 + 0.318933j,
                     -0.0764131 + 0.0695855j])
    assert np.max(np.abs(got - want)) < 1e-6


def test_polar_axis_and_low_l():
    # on the axis only m = 0 is written, with the value sqrt((2l+1)/4pi) (SO3/SO3part.hpp:364-366)
    for l in (0, 1, 3):
        got = ora.spharm(l, np.array([[[0.0], [0.0], [2.5]]], dtype=np.float32))[0, :, 0]
        want = np.zeros(2 * l + 1, dtype=np.complex64)
        want[l] = np.sqrt((2 * l + 1) / (4 * np.pi))
        assert np.allclose(got, want, atol=1e-7)
    # l = 1 closed form: Y_1^0 = sqrt(3/4pi) z, Y_1^{+-1} = -+ sqrt(3/8pi) (x +- iy)
    X = np.random.default_rng(3).standard_normal((2, 3, 5)).astype(np.float32)
    U = X / np.linalg.norm(X, axis=1, keepdims=True)
    got = ora.spharm(1, X)
    assert np.allclose(got[:, 1, :], np.sqrt(3 / (4 * np.pi)) * U[:, 2, :], atol=1e-6)
    assert np.allclose(got[:, 2, :], -np.sqrt(3 / (8 * np.pi)) * (U[:, 0, :] + 1j * U[:, 1, :]), atol=1e-6)
    assert np.allclose(got[:, 0, :], np.sqrt(3 / (8 * np.pi)) * (U[:, 0, :] - 1j * U[:, 1, :]), atol=1e-6)


def test_batch_broadcast_and_scale_invariance():
    X = np.random.default_rng(5).standard_normal((1, 3, 4)).astype(np.float32)
    a = ora.spharm(3, X, batch=3)
    assert a.shape[0] == 3 and np.array_equal(a[0], a[2])
    b = ora.spharm(3, (4.0 * X).astype(np.float32))
    assert np.allclose(a[0], b[0], atol=2e-6)


@pytest.mark.parametrize("l1,l2,l", [(1, 1, 2), (1, 2, 3), (2, 2, 2), (3, 2, 1), (2, 2, 0), (4, 3, 5), (6, 6, 4)])
def test_product_of_harmonics(l1, l2, l):
    """CGproduct(Y_l1(x), Y_l2(x), l) = sqrt((2l1+1)(2l2+1) / (4 pi (2l+1))) <l1 0 l2 0 | l 0> Y_l(x): ties the
    phase convention of the harmonics to that of the coefficients and of the product kernel."""
    X = np.random.default_rng(l1 + 10 * l2).standard_normal((3, 3, 1)).astype(np.float32)
    z = ora.cg_fwd(ora.spharm(l1, X), ora.spharm(l2, X), l)
    c = np.sqrt((2 * l1 + 1) * (2 * l2 + 1) / (4 * np.pi * (2 * l + 1))) * ora.cg_coeff(l1, l2, l, 0, 0)
    assert np.max(np.abs(z - c * ora.spharm(l, X))) < 2e-6
