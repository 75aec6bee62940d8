"""Pins for the SORF / feature / Gram / RFF oracle: closed forms, adjoint identities,
finite differences and the agreement of the reference's two force routes."""
import numpy as np
import pytest
from scipy.linalg import hadamard

from oracle import fchl19, model, sorf
from tests import helpers


@pytest.mark.parametrize("d", [2, 4, 8, 32, 64, 128, 256])
def test_fwht_is_sylvester_hadamard(d):
    rng = np.random.default_rng(d)
    x = rng.normal(size=(3, d))
    assert np.allclose(sorf.fwht(x), x @ hadamard(d).T, rtol=1e-12, atol=1e-12)
    # involution and norm preservation after normalisation
    y = sorf.fwht(x) / np.sqrt(d)
    assert np.allclose(sorf.fwht(y) / np.sqrt(d), x)
    assert np.allclose(np.linalg.norm(y, axis=1), np.linalg.norm(x, axis=1))


def test_fwht_rejects_non_power_of_two():
    with pytest.raises(RuntimeError):
        sorf.fwht(np.zeros((1, 12)))


@pytest.mark.parametrize("T", [1, 2, 3])
def test_sorf_closed_form_and_adjoint(T):
    rng = np.random.default_rng(T)
    A, S, d = 5, 3, 16
    x = rng.normal(size=(A, d))
    D = np.where(rng.uniform(-1, 1, (T, S, d)) > 0, 1.0, -1.0)
    norm = 1.7
    c = sorf.sorf_coefficients(x, D, norm)
    H = hadamard(d) / np.sqrt(d)
    for s in range(S):
        M = np.eye(d)
        for m in range(T):
            M = H @ np.diag(D[m, s]) @ M          # later transforms act on the left
        assert np.allclose(c[:, s, :], norm * x @ M.T)
    y = rng.normal(size=(A, S, d))
    assert np.isclose((c * y).sum(), (x * sorf.sorf_adjoint(y, D, norm)).sum())


def test_cos_features_and_backward_closed_form():
    rng = np.random.default_rng(0)
    A, F, nmol = 7, 24, 3
    c = rng.normal(size=(A, F)) * 3
    b = rng.uniform(0, 2 * np.pi, F)
    idx = np.array([0, 0, 1, 1, 1, 2, 2])
    Z = sorf.cos_features(c, b, idx, nmol)
    for m in range(nmol):
        assert np.allclose(Z[m], np.sqrt(2 / F) * np.cos(c[idx == m] + b).sum(0))
    g = rng.normal(size=(nmol, F))
    gc = sorf.cos_features_backward(g, c, b, idx)
    h = 1e-6
    for (a, f) in [(0, 0), (3, 5), (6, 23)]:
        cp, cm = c.copy(), c.copy()
        cp[a, f] += h
        cm[a, f] -= h
        fd = ((sorf.cos_features(cp, b, idx, nmol) - sorf.cos_features(cm, b, idx, nmol)) * g).sum() / (2 * h)
        assert np.isclose(gc[a, f], fd, rtol=1e-6, atol=1e-9)
    assert np.allclose(sorf.sin_coeffs(c, b), np.sqrt(2 / F) * np.sin(c + b))


def _small_model(T=1):
    prm = fchl19.FCHLParams([1, 6], nRs2=6, nRs3=4, rcut=4.5)
    coords, charges = helpers.benzene_batch(2, seed=0)
    red, D, bias, alpha = helpers.model_weights(2, prm.repsize, 8, 4, ntransforms=T)
    return prm, coords, charges, red, D.astype(np.float64), bias, alpha


@pytest.mark.parametrize("T", [1, 2])
def test_derivative_features_match_fd_and_forces(T):
    prm, coords, charges, red, D, bias, alpha = _small_model(T)
    sigma = 2.0
    X, Z, aid, mid, nat = model.format_batch(coords, charges)
    rows, y = model.sorf_training_rows(X, Z, aid, mid, nat, prm, [1, 6], red, D, bias, sigma,
                                       E=np.array([1.0, 2.0]), F=np.ones((2, 12, 3)))
    B, n = 2, 12
    Zf, G = rows[:B], rows[B:].reshape(B, n, 3, -1)
    # G = -dZ/dR by finite differences of Z (neighbour list frozen)
    h = 1e-5
    for (m, j, x) in [(0, 0, 0), (1, 7, 2), (0, 11, 1)]:
        Xp, Xm = X.copy(), X.copy()
        Xp[m, j, x] += h
        Xm[m, j, x] -= h
        Zp = model.sorf_energy_forces(Xp, Z, aid, mid, nat, prm, [1, 6], red, D, bias, alpha, sigma, forces=False)[2]
        Zm = model.sorf_energy_forces(Xm, Z, aid, mid, nat, prm, [1, 6], red, D, bias, alpha, sigma, forces=False)[2]
        fd = -(Zp[m] - Zm[m]) / (2 * h)
        assert np.allclose(G[m, j, x], fd, rtol=1e-5, atol=1e-7 * np.abs(G).max())
    # the two routes of the reference agree: G.alpha == -dE/dX from the reverse-mode route
    E, Fr, Zf2 = model.sorf_energy_forces(X, Z, aid, mid, nat, prm, [1, 6], red, D, bias, alpha, sigma)
    assert np.allclose(Zf, Zf2)
    assert np.allclose(G @ alpha, Fr, rtol=1e-9, atol=1e-10 * np.abs(Fr).max())
    # targets layout: B energies then B*n*3 forces
    assert y.shape == (B + B * n * 3, 1) and y[0, 0] == 1.0 and y[1, 0] == 2.0 and (y[2:] == 1).all()


def test_training_rows_variants_and_gram():
    rng = np.random.default_rng(2)
    Z = rng.normal(size=(3, 8))
    G = rng.normal(size=(3, 2, 3, 8))
    E = rng.normal(size=3)
    Fo = rng.normal(size=(3, 2, 3))
    r, y = sorf.training_rows(Z, G, E, None)
    assert r.shape == (3, 8) and y.shape == (3, 1)
    r, y = sorf.training_rows(Z, G, None, Fo)
    assert (r[:3] == 0).all() and (y[:3] == 0).all() and np.allclose(r[3:], G.reshape(-1, 8))
    r, y = sorf.training_rows(Z, G, E, Fo)
    ZTZ, ZTy = sorf.gram(r, y)
    assert np.allclose(ZTZ, ZTZ.T)
    assert np.allclose(ZTZ, sum(np.outer(v, v) for v in r))
    assert np.allclose(ZTy[:, 0], sum(v * t for v, t in zip(r, y[:, 0])))
    # feature tiling (kernel.py:78-91,172-181) reproduces the untiled product
    tiles = [r[:, s:s + 3].T @ r for s in range(0, 8, 3)]
    assert np.allclose(np.concatenate(tiles, 0), ZTZ)


def test_regularised_solve_satisfies_the_normal_equations():
    """alpha minimises |Z a - y|^2 + lambda |a|^2: the gradient vanishes, the Cholesky route agrees,
    and for lambda -> 0 with full column rank it is the least-squares solution."""
    rng = np.random.default_rng(4)
    Z = rng.normal(size=(90, 40))
    y = rng.normal(size=(90, 1))
    ZTZ, ZTy = sorf.gram(Z, y)
    lam = 1e-3
    a = sorf.regularised_solve(ZTZ, ZTy, lam)
    grad = Z.T @ (Z @ a - y) + lam * a
    assert np.abs(grad).max() < 1e-10
    L = np.linalg.cholesky(ZTZ + lam * np.eye(40))
    a_chol = np.linalg.solve(L.T, np.linalg.solve(L, ZTy))
    assert np.abs(a - a_chol).max() < 1e-12
    a0 = sorf.regularised_solve(ZTZ, ZTy, 0.0)
    assert np.abs(a0 - np.linalg.lstsq(Z, y, rcond=None)[0]).max() < 1e-10
    assert np.array_equal(ZTZ, Z.T @ Z)                    # the input is not modified


def test_matmul_and_reduce_close_to_fp64():
    rng = np.random.default_rng(3)
    A = rng.normal(size=(16, 200)).astype(np.float32)
    Bm = rng.normal(size=(200, 16)).astype(np.float32)
    C = np.ones((16, 16))
    out = sorf.matmul_and_reduce(A, Bm, C.copy())
    exact = 1.0 + A.astype(np.float64) @ Bm.astype(np.float64)
    assert np.abs(out - exact).max() < 4e-6      # Kahan: error ~ fp32 eps on the result, not ~K eps
    naive = np.zeros((16, 16), dtype=np.float32)
    for k in range(200):
        naive = (naive + A[:, k:k + 1] * Bm[k:k + 1, :]).astype(np.float32)
    assert np.abs(out - exact).max() <= np.abs(1.0 + naive - exact).max()


def test_rff_closed_form_and_forces():
    prm = fchl19.FCHLParams([1, 6], nRs2=6, nRs3=4, rcut=4.5)
    coords, charges = helpers.benzene_batch(2, seed=1)
    red, _, _, _ = helpers.model_weights(2, prm.repsize, 8, 4)
    rng = np.random.default_rng(4)
    Fn = 40
    W = rng.normal(size=(2, 8, Fn)) / (2 * 2.0 ** 2)
    b = rng.uniform(0, 2 * np.pi, (2, Fn))
    alpha = rng.normal(size=Fn)
    X, Z, aid, mid, nat = model.format_batch(coords, charges)
    E, Fr, Zf = model.rff_energy_forces(X, Z, aid, mid, nat, prm, [1, 6], red, W, b, alpha)
    rep, J, _ = model.representation(X, Z, aid, mid, nat, prm, jacobian=True)
    G = np.zeros((2, 12, 3, Fn))
    Zc = np.zeros((2, Fn))
    for ei, e in enumerate([1, 6]):
        mask = Z.astype(int) == e
        idx = np.nonzero(mask)[0]
        sub = sorf.project(rep[mask], red[ei])
        Zc += sorf.rff_features(sub, W[ei], b[ei], idx, 2)
        G += sorf.rff_derivative_features(sub, sorf.project(J[mask], red[ei]), W[ei], b[ei], idx, 2)
    assert np.allclose(Zc, Zf)
    assert np.allclose(G @ alpha, Fr, rtol=1e-9, atol=1e-10 * np.abs(Fr).max())
    h = 1e-5
    Xp, Xm = X.copy(), X.copy()
    Xp[1, 4, 1] += h
    Xm[1, 4, 1] -= h
    Ep = model.rff_energy_forces(Xp, Z, aid, mid, nat, prm, [1, 6], red, W, b, alpha, forces=False)[0]
    Em = model.rff_energy_forces(Xm, Z, aid, mid, nat, prm, [1, 6], red, W, b, alpha, forces=False)[0]
    assert np.isclose(Fr[1, 4, 1], -(Ep - Em).sum() / (2 * h), rtol=1e-5)


def test_rff_normalisation_is_pinned_by_the_gaussian_kernel_identity():
    """Random Fourier features approximate a Gaussian kernel (Rahimi & Recht 2007): for W with
    independent N(0, s^2) entries and b ~ U(0, 2 pi), z(x) = sqrt(2/F) cos(x W + b) satisfies
    E[z(x).z(y)] = exp(-s^2 |x - y|^2 / 2), so z(x).z(x) -> 1.  A wrong feature normalisation
    (sqrt(1/F), 2/F, a missing factor) or a wrong use of W or b moves these by O(1); the sampling
    error at F = 1e5 is sqrt(1/(2F)) = 2.2e-3 for z(x).z(x) and below 3.2e-3 for z(x).z(y):
    the 1e-2 bound below is three of those.  The reference draws W = N(0,1) / (2 sigma^2)
    (models/random_features.py:54), i.e. s = 1 / (2 sigma^2)."""
    rng = np.random.default_rng(42)
    F, d, sigma = 100000, 6, 0.6
    s = 1.0 / (2.0 * sigma ** 2)
    W = rng.normal(size=(d, F)) * s
    b = rng.uniform(0.0, 2.0 * np.pi, F)
    x = rng.normal(size=(5, d)) * 0.5
    # one atom per molecule: row a of the feature matrix is z(x_a)
    Z = sorf.rff_features(x, W, b, np.arange(5), 5)
    K = Z @ Z.T
    d2 = ((x[:, None, :] - x[None, :, :]) ** 2).sum(-1)
    expect = np.exp(-0.5 * s * s * d2)
    assert expect.min() < 0.5                      # the test points are not all on top of each other
    assert np.abs(np.diag(K) - 1.0).max() < 1e-2
    assert np.abs(K - expect).max() < 1e-2
    # two atoms in one molecule add their feature vectors (random_features_kernel.cu:28-40)
    Z2 = sorf.rff_features(x[:2], W, b, np.array([0, 0]), 1)
    assert np.allclose(Z2[0], Z[0] + Z[1])
    # the force-feature rows are minus the derivative of the features along the given rows
    grad = np.eye(d).reshape(1, 2, 3, d)             # row (j, c) of the "Jacobian" is the unit vector 3 j + c
    G = sorf.rff_derivative_features(x[:1], grad, W, b, np.array([0]), 1)
    h = 1e-6
    for k in (0, 4):
        xp, xm = x[:1].copy(), x[:1].copy()
        xp[0, k] += h
        xm[0, k] -= h
        fd = (sorf.rff_features(xp, W, b, np.array([0]), 1) - sorf.rff_features(xm, W, b, np.array([0]), 1)) / (2 * h)
        assert np.abs(G[0, k // 3, k % 3] + fd[0]).max() < 1e-8
