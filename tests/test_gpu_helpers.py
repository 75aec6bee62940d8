"""GPU parity of the Python-level helpers a user of the reference imports directly: the autograd
wrappers and free functions of features/SORF.py and the per-element reductor fit of
representations/dimensionality_reduction.py, against the fp64 oracle."""
import numpy as np
import pytest
import torch

from oracle import sorf

pytestmark = pytest.mark.gpu

REL = 1e-5


def dev():
    return torch.device("cuda:0")


def close(got, ref, rel, what=""):
    got = got.detach().double().cpu().numpy()
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    scale = max(np.abs(ref).max(), 1e-30)
    err = np.abs(got - ref).max()
    assert err <= rel * scale, "%s: max abs err %.3e over scale %.3e" % (what, err, scale)


def case(seed, A=11, d=64, S=5, T=2, nmol=4, n=3):
    rng = np.random.default_rng(seed)
    x = rng.normal(size=(A, d)).astype(np.float32)
    D = np.where(rng.uniform(-1, 1, (T, S, d)) > 0, 1.0, -1.0).astype(np.float32)
    b = rng.uniform(0, 2 * np.pi, S * d).astype(np.float32)
    idx = np.sort(rng.integers(0, nmol, A)).astype(np.int32)
    u = rng.normal(size=(A, n, 3, d)).astype(np.float32)
    return x, D, b, idx, u


def test_autograd_wrappers_forward_and_gradient():
    """SORFTransformCuda -> CosFeatures -> a linear functional: value and d/dx against the oracle's
    forward and adjoint chain (features/SORF.py:15-80)."""
    from qml_lightning_amd.features.SORF import CosFeatures, SORFTransformCuda
    x, D, b, idx, _ = case(1)
    A, d = x.shape
    S, nmol, norm = D.shape[1], 4, 1.3
    w = np.random.default_rng(2).normal(size=(nmol, S * d))
    xt = torch.tensor(x, device=dev(), requires_grad=True)
    coeffs = SORFTransformCuda.apply(xt, torch.tensor(D, device=dev()), norm, D.shape[0])
    assert coeffs.shape == (A, S, d)
    Z = CosFeatures.apply(coeffs.view(A, -1), torch.tensor(b, device=dev()), nmol, torch.tensor(idx, device=dev()))
    loss = (Z.double() * torch.tensor(w, device=dev())).sum()
    loss.backward()
    c_ref = sorf.sorf_coefficients(x, D, norm)
    close(coeffs, c_ref, REL, "coefficients")
    close(Z, sorf.cos_features(c_ref.reshape(A, -1), b, idx, nmol), REL, "features")
    g_c = sorf.cos_features_backward(w, c_ref.reshape(A, -1), b, idx)
    close(xt.grad, sorf.sorf_adjoint(g_c.reshape(A, S, d), D, norm), 1e-4, "gradient")


def test_per_element_reductor_fit():
    """Columns = leading left singular vectors of the element's rows: orthonormal, and they span
    the same subspace as numpy's SVD of the same rows (all rows are used while there are at most
    512 of them, so the random choice does not matter here)."""
    from qml_lightning_amd.representations.dimensionality_reduction import get_reductors, project_representation
    rng = np.random.default_rng(8)
    R, npcas = 40, 6
    decay = np.exp(-0.5 * np.arange(R))
    gto = (rng.normal(size=(3, 50, R)) * decay).astype(np.float32)
    charges = rng.choice([1.0, 6.0, 0.0], size=(3, 50))
    red = get_reductors(torch.tensor(gto, device=dev()), torch.tensor(charges, device=dev()), npcas, [1, 6, 8])
    assert set(red) == {1, 6}                        # no atom of element 8: no entry
    for e in (1, 6):
        U = red[e].double().cpu().numpy()
        assert U.shape == (R, npcas)
        assert np.abs(U.T @ U - np.eye(npcas)).max() < 1e-5
        rows = gto[charges == e].astype(np.float64)
        Uref = np.linalg.svd(rows.T, full_matrices=False)[0][:, :npcas]
        assert np.abs(U @ U.T - Uref @ Uref.T).max() < 1e-4
        proj = project_representation(torch.tensor(rows, device=dev()).float(), red[e])
        close(proj.abs(), np.abs(rows @ Uref), 1e-4, "projection up to the sign of each column")


def test_util_ops_free_functions():
    """utils/util_ops.format_data (ragged lists, one molecule, same_mol) gives the layout the
    model's own format_data gives, and the representation computed from it agrees; the
    self-energy fit recovers exact per-element energies."""
    from qml_lightning_amd.models.hadamard_features import HadamardFeaturesModel
    from qml_lightning_amd.representations.FCHL import FCHLCuda
    from qml_lightning_amd.utils import synthetic, util_ops
    coords, charges = synthetic.ragged_batch(9, seed=4)
    coords = [c.astype(np.float32) for c in coords]
    rng = np.random.default_rng(0)
    E = rng.normal(size=9)
    Fs = [rng.normal(size=c.shape) for c in coords]
    rep = FCHLCuda(species=np.array([1, 6, 7, 8, 9]))
    m = HadamardFeaturesModel(rep=rep, elements=np.array([1, 6, 7, 8, 9]), npcas=64, nstacks=2)
    mine = m.format_data(coords, charges, E=E, F=Fs)
    free = util_ops.format_data(coords, charges, E=E, F=Fs)
    for k in ('coordinates', 'charges', 'natom_counts', 'atomIDs', 'molIDs', 'energies', 'forces', 'cells', 'inv_cells'):
        assert free[k].dtype == mine[k].dtype and torch.equal(free[k], mine[k]), k
    one = util_ops.format_data(coords[2], charges[2])
    assert one['coordinates'].shape == (1, len(charges[2]), 3) and one['energies'] is None
    assert one['cells'].shape == (0, 3, 3)
    # same composition: whole arrays
    xs, qs = synthetic.fixed_composition_batch(synthetic.ASPIRIN, 5, seed=2)
    X, Q = np.asarray(xs, dtype=np.float32), np.asarray(qs)
    same = util_ops.format_data(X, Q, same_mol=True)
    lists = util_ops.format_data(list(X), list(Q))
    for k in ('coordinates', 'charges', 'natom_counts', 'atomIDs', 'molIDs'):
        assert same[k].dtype == lists[k].dtype and torch.equal(same[k], lists[k]), k
    assert 'energies' not in same
    rep3 = FCHLCuda(species=np.array([1, 6, 8]))
    ra = rep3.get_representation(same['coordinates'], same['charges'], same['atomIDs'], same['molIDs'], same['natom_counts'],
                                 same['cells'], same['inv_cells'])
    rb = rep3.get_representation(lists['coordinates'], lists['charges'], lists['atomIDs'], lists['molIDs'],
                                 lists['natom_counts'], lists['cells'], lists['inv_cells'])
    assert torch.equal(ra, rb)
    # self energies: E = sum over atoms of a per-element constant
    true = {1: -0.5, 6: -37.8, 7: -54.6, 8: -75.0, 9: -99.7}
    Es = [sum(true[int(z)] for z in q) for q in charges]
    se = util_ops.calculate_self_energy(charges, Es, torch.tensor([1, 6, 7, 8, 9]))
    assert se.shape == (10,) and se.dtype == torch.float64
    for z, v in true.items():
        assert abs(float(se[z]) - v) < 1e-6 * abs(v) + 1e-8, (z, float(se[z]), v)
