"""Pins for the FCHL19 oracle that do not retype its formulas: finite differences,
sum rules, invariances, brute force, and a hand-evaluated 3-atom case."""
import numpy as np
import pytest

from oracle import fchl19, model
from tests import helpers


def _rep(coords, charges, prm, jac=False, cell=None, inv_cell=None):
    X, Z, aid, mid, nat = model.format_batch(coords, charges)
    return model.representation(X, Z, aid, mid, nat, prm, cell, inv_cell, jacobian=jac), (X, Z, aid, mid, nat)


def test_neighbours_bruteforce():
    rng = np.random.default_rng(5)
    coords = [rng.uniform(0, 6, (n, 3)) for n in (3, 9, 17)]
    X, Z, aid, mid, nat = model.format_batch(coords, [np.ones(len(c)) for c in coords])
    rcut = 3.0
    cnt, nl = fchl19.neighbours(X, nat, rcut)
    for m, c in enumerate(coords):
        for i in range(len(c)):
            exp = [j for j in range(len(c)) if j != i and np.linalg.norm(c[i] - c[j]) < rcut]
            assert cnt[m, i] == len(exp)
            assert list(nl[m, i, :len(exp)]) == exp
            assert (nl[m, i, len(exp):] == -1).all()
    assert (cnt[0, 3:] == 0).all()


def test_minimum_image_bruteforce():
    rng = np.random.default_rng(6)
    cell = np.array([[5.0, 0.0, 0.0], [0.4, 4.5, 0.0], [0.3, -0.2, 6.0]]).T  # columns = box vectors
    inv = np.linalg.inv(cell)
    d = rng.uniform(-4, 4, (50, 3))
    mi = fchl19.pbc_drij(d, cell, inv)
    shifts = np.array([[a, b, c] for a in (-2, -1, 0, 1, 2) for b in (-2, -1, 0, 1, 2) for c in (-2, -1, 0, 1, 2)])
    for v, w in zip(d, mi):
        # the result is a lattice translate of v ...
        s = inv @ (v - w)
        assert np.allclose(s, np.round(s), atol=1e-9)
        # ... with fractional coordinates in [-1/2, 1/2]
        assert (np.abs(inv @ w) <= 0.5 + 1e-12).all()


def test_three_atom_hand_case():
    """One C centre with two H neighbours at right angles: every factor evaluated by hand."""
    prm = fchl19.FCHLParams([1, 6], rcut=4.0, nRs2=3, nRs3=2, eta2=0.4, eta3=1.5,
                            two_body_decay=2.0, three_body_weight=3.0, three_body_decay=0.5)
    a, b = 1.1, 1.3
    coords = [np.array([[0.0, 0, 0], [a, 0, 0], [0, b, 0]])]
    (rep, _), _ = _rep(coords, [np.array([6, 1, 1])], prm)
    r = rep[0, 0]
    fc = lambda x: 0.5 * (np.cos(np.pi * x / 4.0) + 1)
    # two-body, element H (index 0): sum over both neighbours of lognormal pdf(Rs; mu, sigma) / r^2 * fc
    exp2 = np.zeros(3)
    for x in (a, b):
        s2 = np.log(1 + 0.4 / x ** 2)
        mu = np.log(x) - 0.5 * s2
        pdf = np.exp(-(np.log(prm.Rs2) - mu) ** 2 / (2 * s2)) / (prm.Rs2 * np.sqrt(2 * np.pi * s2))
        exp2 += pdf / x ** 2 * fc(x)
    assert np.allclose(r[0:3], exp2, rtol=1e-12)
    assert np.allclose(r[3:6], 0)           # no C neighbours
    # three-body: pair (H,H) -> p=q=0 -> offset ns*nRs2 + 0
    c = np.hypot(a, b)
    cos_i, cos_j, cos_k = 0.0, a / c, b / c
    ksi = np.sqrt(1.5 / np.pi) * 3.0 * (1 + 3 * cos_i * cos_j * cos_k) / (a * b * c) ** 0.5
    rad = np.exp(-1.5 * (0.5 * (a + b) - prm.Rs3) ** 2) * fc(a) * fc(b)
    z = 2 * np.exp(-np.pi ** 2 / 2)
    off = 2 * 3
    assert np.allclose(r[off:off + 4:2], rad * z * 0.0 * ksi, atol=1e-15)      # cos(90 deg) = 0
    assert np.allclose(r[off + 1:off + 4:2], rad * z * 1.0 * ksi, rtol=1e-12)  # sin(90 deg) = 1
    assert np.allclose(r[off + 4:], 0)
    # H atom 1 sees C (type 1) and H (type 0): pair (0,1) -> offset ns*nRs2 + 2*nRs3*(0 + 1 + 0)
    r1 = rep[0, 1]
    nz = np.nonzero(np.abs(r1[6:]) > 0)[0]
    assert nz.min() >= 4 and nz.max() < 8


def test_invariances():
    prm = fchl19.FCHLParams([1, 6, 8])
    coords, charges = helpers.fixed_composition_batch(helpers.ASPIRIN, 1, seed=1)
    (rep, _), _ = _rep(coords, charges, prm)
    # rotation + translation
    rng = np.random.default_rng(3)
    Q, _ = np.linalg.qr(rng.normal(size=(3, 3)))
    (rep2, _), _ = _rep([coords[0] @ Q.T + rng.normal(size=3)], charges, prm)
    assert np.allclose(rep, rep2, rtol=1e-9, atol=1e-12)
    # permutation of atoms permutes rows
    perm = rng.permutation(len(charges[0]))
    (rep3, _), _ = _rep([coords[0][perm]], [charges[0][perm]], prm)
    assert np.allclose(rep[0][perm], rep3[0], rtol=1e-9, atol=1e-12)


@pytest.mark.parametrize("species,charges,seed", [([1, 6], None, 0), ([1, 6, 7, 8], np.array([6, 1, 7, 8, 1, 6, 1]), 4)])
def test_jacobian_vs_finite_differences(species, charges, seed):
    prm = fchl19.FCHLParams(species, nRs2=6, nRs3=5, rcut=4.5)
    if charges is None:
        coords, ch = helpers.benzene_batch(1, seed)
    else:
        coords, ch = helpers.fixed_composition_batch(charges, 1, seed, box=3.5)
    (rep, J, ctx), (X, Z, aid, mid, nat) = _rep(coords, ch, prm, jac=True)
    types, nlist, nneigh = ctx
    n = X.shape[1]
    h = 1e-5
    Jfd = np.zeros_like(J)
    for j in range(n):
        for x in range(3):
            Xp, Xm = X.copy(), X.copy()
            Xp[0, j, x] += h
            Xm[0, j, x] -= h
            rp = fchl19.forward(Xp, types, aid, mid, nlist, nneigh, prm)
            rm = fchl19.forward(Xm, types, aid, mid, nlist, nneigh, prm)
            Jfd[0, :, j, x, :] = (rp[0] - rm[0]) / (2 * h)
    scale = np.abs(Jfd).max()
    assert np.abs(J - Jfd).max() < 1e-7 * scale
    # translation sum rule
    assert np.abs(J.sum(axis=2)).max() < 1e-10 * scale
    # VJP is the contraction of the Jacobian
    g = np.random.default_rng(1).normal(size=rep.shape)
    v = fchl19.vjp(g, X, types, aid, mid, nlist, nneigh, prm)
    assert np.allclose(v, np.einsum("mif,mijxf->mjx", g, Jfd), rtol=1e-6, atol=1e-7 * scale)


def test_jacobian_pbc_finite_differences():
    prm = fchl19.FCHLParams([1, 8], nRs2=4, nRs3=3, rcut=2.4)
    rng = np.random.default_rng(8)
    cellm = np.array([[5.0, 0.0, 0.0], [0.5, 5.2, 0.0], [0.2, 0.3, 4.9]]).T
    coords = [helpers.random_geometry(rng, 6, 4.8, 1.2)]
    ch = [np.array([8, 1, 1, 8, 1, 1])]
    cell, inv = cellm[None], np.linalg.inv(cellm)[None]
    (rep, J, ctx), (X, Z, aid, mid, nat) = _rep(coords, ch, prm, jac=True, cell=cell, inv_cell=inv)
    types, nlist, nneigh = ctx
    # the periodic images matter in this cell: more neighbours than the open molecule has
    cnt_open, _ = fchl19.neighbours(X, nat, prm.rcut)
    assert nneigh.sum() > cnt_open.sum()
    h = 1e-5
    for j in (0, 3):
        for x in range(3):
            Xp, Xm = X.copy(), X.copy()
            Xp[0, j, x] += h
            Xm[0, j, x] -= h
            rp = fchl19.forward(Xp, types, aid, mid, nlist, nneigh, prm, cell, inv)
            rm = fchl19.forward(Xm, types, aid, mid, nlist, nneigh, prm, cell, inv)
            fd = (rp[0] - rm[0]) / (2 * h)
            assert np.abs(J[0, :, j, x, :] - fd).max() < 1e-6 * max(1.0, np.abs(fd).max())
