"""Host-side logic that needs no GPU: batch formatting, targets layout, model attributes
and TorchScript compilation of the forward methods."""
import os

import numpy as np
import pytest
import torch

from oracle import model as omodel


def _model(fused=True):
    from qml_lightning_amd.models.hadamard_features import HadamardFeaturesModel
    from qml_lightning_amd.representations.FCHL import FCHLCuda
    rep = FCHLCuda(species=np.array([1, 6, 8]))
    return HadamardFeaturesModel(rep=rep, elements=np.array([1, 6, 8]), ntransforms=1, sigma=2.0, npcas=128,
                                 nstacks=4, fused=fused)


def test_fchl_hyperparameter_tensors_match_reference_layout():
    from qml_lightning_amd.representations.FCHL import FCHLCuda
    rep = FCHLCuda(species=np.array([1, 6, 7, 8]), eta3=2.7, three_body_weight=13.4)
    assert rep.get_repsize() == 4 * 24 + 4 * 5 * 20
    # FCHL.py:35 -- the weight handed to the kernels carries sqrt(eta3/pi)
    assert np.isclose(float(rep.three_body_weight), np.sqrt(2.7 / np.pi) * 13.4)
    assert np.allclose(rep.Rs2.cpu().numpy(), np.linspace(0, 6, 25)[1:])
    assert rep.species.dtype == torch.float32 and rep.eta2.dim() == 0


def test_format_data_matches_oracle_layout():
    m = _model()
    rng = np.random.default_rng(0)
    coords = [rng.normal(size=(n, 3)) for n in (3, 5, 2)]
    charges = [np.array([1, 6, 8]), np.array([6, 6, 1, 1, 8]), np.array([1, 1])]
    E = [1.0, 2.0, 3.0]
    F = [rng.normal(size=c.shape) for c in coords]
    d = m.format_data(coords, charges, E=E, F=F)
    X, Z, aid, mid, nat = omodel.format_batch(coords, charges)
    assert np.allclose(d['coordinates'].cpu().numpy(), X.astype(np.float32))
    assert (d['charges'].cpu().numpy() == Z).all() and d['charges'].dtype == torch.float32
    assert (d['atomIDs'].cpu().numpy() == aid).all() and d['atomIDs'].dtype == torch.int32
    assert (d['molIDs'].cpu().numpy() == mid).all() and (d['natom_counts'].cpu().numpy() == nat).all()
    assert d['forces'].shape == (3, 5, 3) and d['forces'].dtype == torch.float64
    assert (d['forces'][0, 3:] == 0).all()
    assert d['cells'].shape == (0, 3, 3)
    flat = Z.reshape(-1).astype(int)
    # a training batch carries the per-element atom counts (the index itself is a device sort)
    assert d['element_counts'] == {e: int((flat == e).sum()) for e in (1, 6, 8)}
    for e in (1, 6, 8):
        assert (m._element_index(d, d['charges'], e).cpu().numpy() == np.nonzero(flat == e)[0]).all()
    t = m._targets(d, 3, True, True)
    assert t.shape == (3 + 3 * 5 * 3, 1) and t[1, 0] == 2.0
    assert np.allclose(t[3:, 0].cpu().numpy(), d['forces'].cpu().numpy().reshape(-1))
    t = m._targets(d, 3, False, True)
    assert (t[:3] == 0).all()
    # nested Python lists give the same tensors; a predict batch carries no per-element index lists
    d2 = m.format_data([c.tolist() for c in coords], [q.tolist() for q in charges])
    for key in ("coordinates", "charges", "atomIDs", "molIDs", "natom_counts"):
        assert torch.equal(d2[key], d[key]), key
    assert 'element_counts' not in d2 and d2['energies'] is None and d2['forces'] is None
    # the same batch as one zero-padded array pair with targets: identical tensors, self energies included
    Xp, Qp, Fp = np.zeros((3, 5, 3)), np.zeros((3, 5)), np.zeros((3, 5, 3))
    for k, (c, q, f) in enumerate(zip(coords, charges, F)):
        Xp[k, :len(q)], Qp[k, :len(q)], Fp[k, :len(q)] = c, q, f
    Fp[0, 4] = 7.0                                    # a target in a padded slot is dropped
    d3 = m.format_data(Xp, Qp, E=np.array(E), F=Fp)
    for key in ("coordinates", "charges", "atomIDs", "molIDs", "natom_counts", "energies", "forces"):
        assert d3[key].dtype == d[key].dtype and torch.equal(d3[key], d[key]), key
    assert d3['element_counts'] == d['element_counts']
    m.self_energy = torch.tensor([0.0, -0.5, 0, 0, 0, 0, -38.0, 0, -75.0], dtype=torch.float64)
    m.set_subtract_self_energies(True)
    m.set_convert_hartree2kcal(True)
    dl = m.format_data(coords, charges, E=E, F=F)
    dp = m.format_data(Xp, Qp, E=np.array(E), F=Fp)
    assert torch.allclose(dl['energies'], dp['energies'], rtol=1e-14, atol=0) and torch.equal(dl['forces'], dp['forces'])
    m.set_subtract_self_energies(False)
    m.set_convert_hartree2kcal(False)
    with pytest.raises(RuntimeError, match="real atoms first"):
        m.format_data(Xp[:, ::-1].copy(), Qp[:, ::-1].copy())
    # the fallback for rows that do not stack directly (a flattened force array)
    rows = m._concat_rows([np.arange(6.0), np.arange(9.0).reshape(3, 3)], 3, np.float64)
    assert rows.shape == (5, 3) and rows[1, 0] == 3.0 and rows[2, 1] == 1.0


def test_self_energy_subtraction_and_unit_conversion():
    m = _model()
    Q = [np.array([1, 1, 8]), np.array([6, 1, 1, 1, 1]), np.array([8, 8]), np.array([6, 8])]
    beta = {1: -0.5, 6: -37.8, 8: -75.0}
    E = [sum(beta[int(q)] for q in qs) for qs in Q]
    m.calculate_self_energy(Q, E)
    for e, v in beta.items():
        assert np.isclose(float(m.self_energy[e]), v, atol=1e-8)
    m.set_subtract_self_energies(True)
    d = m.format_data([np.zeros((len(q), 3)) for q in Q], Q, E=E)
    assert np.allclose(d['energies'].cpu().numpy(), 0.0, atol=1e-8)


def test_forward_compiles_to_torchscript_with_the_reference_operator_names():
    for fused in (True, False):
        s = torch.jit.script(_model(fused))
        code = s.code + s.rep.code
        assert "ops.qml_lightning_fchl.fchl_forwards" in code
        if fused:
            assert "ops.qml_lightning_sorf.fchl_sorf_energy" in code      # the whole chain, one operator
        else:
            assert "ops.qml_lightning_sorf.get_SORF_coefficients" in code
            assert "ops.qml_lightning_sorf.get_cos_features" in code
    m = _model(True)
    m.separate_ops = True                                                 # the fused route operator by operator
    code = torch.jit.script(m).code
    for name in ("sort_by_type", "project_typed", "sorf_energy_sorted"):
        assert "ops.qml_lightning_sorf." + name in code


def test_free_self_energy_fit_matches_the_model_method():
    """utils/util_ops.calculate_self_energy (util_ops.py:10-53) against exact per-element energies
    and against BaseKernel.calculate_self_energy on the same data (host only)."""
    import torch
    from qml_lightning_amd.utils import util_ops
    rng = np.random.default_rng(3)
    true = {1: -0.6, 6: -38.1, 8: -75.2}
    Q = [rng.choice([1, 6, 8], size=int(rng.integers(3, 12))) for _ in range(40)]
    E = [sum(true[int(z)] for z in q) for q in Q]
    se = util_ops.calculate_self_energy(Q, E, torch.tensor([1, 6, 8]))
    assert se.dtype == torch.float64 and se.shape == (9,)
    for z, v in true.items():
        assert abs(float(se[z]) - v) <= 1e-9 * abs(v)
    assert float(se[[0, 2, 3, 4, 5, 7]].abs().max()) == 0.0


def test_small_integer_division_through_a_float_reciprocal_is_exact():
    """The FCHL19 kernels divide small non-negative integers as int((x + 0.5f) * rcp(d)) with the
    1-ulp hardware reciprocal (csrc/fchl19.hip, idiv_small).  Emulated here in fp32 with the
    reciprocal pushed one ulp either way: equal to x // d over the range the kernels use
    (lanes, triple counts, bin items: below 2^17; divisors up to 128)."""
    x = np.arange(0, 1 << 17, dtype=np.int64)
    xf = x.astype(np.float32) + np.float32(0.5)
    for d in range(1, 129):
        r0 = np.float32(1.0) / np.float32(d)
        for r in (np.nextafter(r0, np.float32(0)), r0, np.nextafter(r0, np.float32(2))):
            q = (xf * r).astype(np.int64)
            assert np.array_equal(q, x // d), d


def test_rff_model_draws_its_basis_as_the_reference_does():
    """W = N(0, 1) / (2 sigma^2) per element and feature, b ~ U(0, 2 pi)
    (models/random_features.py:38,54-55): sample moments of a 16 x 4096 draw per element."""
    from qml_lightning_amd.models.random_features import RandomFourrierFeaturesModel
    from qml_lightning_amd.representations.FCHL import FCHLCuda
    np.random.seed(3)
    rep = FCHLCuda(species=np.array([1, 6, 8]))
    for sigma in (2.0, 0.7):
        m = RandomFourrierFeaturesModel(rep=rep, elements=np.array([1, 6, 8]), sigma=sigma, nstacks=256, npcas=16)
        assert m.W.shape == (3, 16, 4096) and m.b.shape == (3, 4096) and m.W.dtype == torch.float32
        s = 1.0 / (2.0 * sigma ** 2)
        for e in range(3):
            W = m.W[e].double().cpu().numpy()
            b = m.b[e].double().cpu().numpy()
            n = W.size
            assert abs(W.std() - s) < 4 * s / np.sqrt(2 * n)          # 4 sigma of the sample std
            assert abs(W.mean()) < 4 * s / np.sqrt(n)
            assert b.min() >= 0.0 and b.max() < 2 * np.pi + 1e-6
            assert abs(b.mean() - np.pi) < 4 * (2 * np.pi / np.sqrt(12)) / np.sqrt(b.size)
            assert abs(b.std() - 2 * np.pi / np.sqrt(12)) < 0.05
        assert np.isclose(m.feature_normalisation, np.sqrt(2.0 / 4096))
        assert not np.allclose(m.W[0].cpu().numpy(), m.W[1].cpu().numpy())        # a draw of its own per element


def test_model_species_for_the_element_sort():
    """The one-operator predict chain indexes reductors / diagonals / bias by the MODEL's element
    list; the representation indexes its bins by ITS species list.  Equal lists: an empty tensor
    (the chain reuses the representation's element types); a subset or another order: the model's
    own list travels with the call."""
    from qml_lightning_amd.models.hadamard_features import HadamardFeaturesModel, model_species_for_sort
    from qml_lightning_amd.models.random_features import RandomFourrierFeaturesModel
    from qml_lightning_amd.representations.FCHL import FCHLCuda
    rep = FCHLCuda(species=np.array([1, 6, 7, 8]))
    same = HadamardFeaturesModel(rep=rep, elements=np.array([1, 6, 7, 8]), ntransforms=1, npcas=16, nstacks=2)
    assert same.sort_species.numel() == 0
    sub = HadamardFeaturesModel(rep=rep, elements=np.array([1, 6, 8]), ntransforms=1, npcas=16, nstacks=2)
    assert sub.sort_species.tolist() == [1.0, 6.0, 8.0] and sub.reductors.shape[0] == 3
    perm = RandomFourrierFeaturesModel(rep=rep, elements=np.array([8, 1, 6, 7]), nstacks=2, npcas=64)
    assert perm.sort_species.tolist() == [8.0, 1.0, 6.0, 7.0]
    assert model_species_for_sort(torch.tensor([1.0, 6.0]), None).tolist() == [1.0, 6.0]
    assert "sort_species" in torch.jit.script(sub).code


def test_closed_form_pair_unranking_is_exact():
    """The FCHL19 kernels number the pairs j < k of a neighbour list k-major, t = k (k - 1) / 2 + j,
    and recover (j, k) from t in fp32 with no correction step: k = int(1/2 + sqrt(2 t + 1.25)),
    j = t - k (k - 1) / 2 (csrc/fchl19.hip, unrank_pair_kmajor).  Emulated here in fp32 with the
    square root pushed up to two ulps either way, for every t below 2^20."""
    t = np.arange(0, 1 << 20, dtype=np.int64)
    tf = t.astype(np.float32)
    kk = ((1 + np.sqrt(1 + 8 * t.astype(np.float64))) // 2).astype(np.int64)
    kk = np.where(kk * (kk - 1) // 2 > t, kk - 1, kk)
    kk = np.where((kk + 1) * kk // 2 <= t, kk + 1, kk)
    jj = t - kk * (kk - 1) // 2
    assert (jj >= 0).all() and (jj < kk).all()
    f32 = np.float32
    for push in (-2, -1, 0, 1, 2):
        sq = np.sqrt((f32(2) * tf + f32(1.25)).astype(np.float32)).astype(np.float32)
        for _ in range(abs(push)):
            sq = np.nextafter(sq, f32(np.inf if push > 0 else -np.inf)).astype(np.float32)
        k = (f32(0.5) + sq).astype(np.float32).astype(np.int64)       # conversion truncates
        assert np.array_equal(k, kk) and np.array_equal(t - k * (k - 1) // 2, jj), push


def test_gram_tile_map_meets_every_tile_once_and_balances_the_xcds(tmp_path):
    """tests/cpp/check_gram_tiles.cpp walks the Gram kernel's workgroup-id -> tile map (the header the
    kernel and its launch use) for 1..140 tiles per edge: every tile on or above the diagonal exactly
    once, nothing below it, XCD shares within one tile of each other for whole super-tiles; the full
    mode every tile once."""
    import shutil
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    if shutil.which("g++") is None:
        pytest.skip("needs g++")
    exe = str(tmp_path / "check_gram_tiles")
    subprocess.run(["g++", "-O2", "-std=c++17", "-I", os.path.join(root, "qml_lightning_amd", "csrc"),
                    os.path.join(root, "tests", "cpp", "check_gram_tiles.cpp"), "-o", exe], check=True)
    out = subprocess.run([exe], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr
    assert out.stdout.startswith("ok")


def test_rff_fused_true_refuses_a_width_without_a_fused_kernel():
    from qml_lightning_amd.models.random_features import RandomFourrierFeaturesModel
    from qml_lightning_amd.representations.FCHL import FCHLCuda
    rep = FCHLCuda(species=np.array([1, 6]))
    with pytest.raises(ValueError, match="fused kernel exists for npcas 64 or 128"):
        RandomFourrierFeaturesModel(rep=rep, elements=np.array([1, 6]), nstacks=2, npcas=256, fused=True)
    auto = RandomFourrierFeaturesModel(rep=rep, elements=np.array([1, 6]), nstacks=2, npcas=256)
    assert auto.fused is False
    assert RandomFourrierFeaturesModel(rep=rep, elements=np.array([1, 6]), nstacks=2, npcas=64).fused is True
