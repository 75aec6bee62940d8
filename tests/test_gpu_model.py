"""GPU parity at the model level: the reference's Python API (FCHLCuda,
HadamardFeaturesModel, RandomFourrierFeaturesModel, torch.ops, TorchScript, autograd
forces, build_Z_components) against the fp64 oracle and the reference's known-answer vector."""
import os

import numpy as np
import pytest
import torch

from oracle import model as omodel
from oracle import sorf as osorf
from tests import helpers
from tests.test_gpu_kernels import REL_EF, REL_REP, close, dev, make_batch, oracle_prm, t32, ti32

pytestmark = pytest.mark.gpu


def build_sorf_model(species, npcas, nstacks, ntransforms=1, sigma=2.0, fused=True, seed=10, **repkw):
    from qml_lightning_amd.models.hadamard_features import HadamardFeaturesModel
    from qml_lightning_amd.representations.FCHL import FCHLCuda
    rep = FCHLCuda(species=np.array(species), **repkw)
    m = HadamardFeaturesModel(rep=rep, elements=np.array(species), ntransforms=ntransforms, sigma=sigma,
                              llambda=1e-5, npcas=npcas, nstacks=nstacks, nbatch_train=4, nbatch_test=5, fused=fused)
    red, D, bias, alpha = helpers.model_weights(len(species), rep.get_repsize(), npcas, nstacks, ntransforms, seed)
    m.reductors = t32(red)
    m.Dmat = t32(D)
    m.bias = t32(bias)
    m.alpha = torch.tensor(alpha, device=dev())
    m.is_trained = True
    return m, (red, D.astype(np.float64), bias, alpha.astype(np.float32).astype(np.float64))


def build_rff_model(species, npcas, nstacks, seed=3):
    from qml_lightning_amd.models.random_features import RandomFourrierFeaturesModel
    from qml_lightning_amd.representations.FCHL import FCHLCuda
    rep = FCHLCuda(species=np.array(species))
    np.random.seed(seed)
    m = RandomFourrierFeaturesModel(rep=rep, elements=np.array(species), sigma=3.0, llambda=1e-5, npcas=npcas,
                                    nstacks=nstacks, nbatch_train=4, nbatch_test=5)
    red, _, _, alpha = helpers.model_weights(len(species), rep.get_repsize(), npcas, nstacks)
    m.reductors = t32(red)
    m.alpha = torch.tensor(alpha, device=dev())
    m.is_trained = True
    return m, red


def inputs(X, Z, aid, mid, nat):
    return t32(X), t32(Z), ti32(aid), ti32(mid), ti32(nat)


def test_reference_known_answer_aspirin(kat):
    """unit_tests/models/unit_test_sorf.py of the reference, run through this library."""
    from qml_lightning_amd.models.hadamard_features import HadamardFeaturesModel
    from qml_lightning_amd.representations.FCHL import FCHLCuda
    d = kat
    for fused in (True, False):
        rep = FCHLCuda(species=np.array([1, 6, 8]), rcut=6.0, nRs2=24, nRs3=22, eta2=0.28, eta3=3.2,
                       two_body_decay=2.3, three_body_weight=18.8, three_body_decay=0.65)
        rep.three_body_weight = torch.tensor(float(d["three_body_weight"]))
        assert np.allclose(rep.Rs2.cpu().numpy(), d["Rs2"]) and np.allclose(rep.Rs3.cpu().numpy(), d["Rs3"])
        m = HadamardFeaturesModel(rep=rep, elements=np.array([1, 6, 8]), ntransforms=1, sigma=2.0, llambda=1e-5,
                                  npcas=128, nstacks=128, fused=fused)
        m.reductors = t32(d["reductors"])
        m.Dmat = t32(d["Dmat"].astype(np.float32))
        m.bias = t32(d["bias"])
        m.alpha = torch.tensor(d["alpha"], device=dev())
        X = t32(d["coordinates"]).unsqueeze(0)
        X.requires_grad = True
        Z = t32(d["charges"]).unsqueeze(0)
        n = d["coordinates"].shape[0]
        E = m.forward(X, Z, torch.arange(n, dtype=torch.int32, device=dev()),
                      torch.zeros(n, dtype=torch.int32, device=dev()), ti32([n]))
        F, = torch.autograd.grad(-E.sum(), X)
        total = d["self_energy"][d["charges"]].sum() + E.item()
        assert np.isclose(float(d["ref_energy"]), total)                       # unit_test_sorf.py:100
        assert abs(total - float(d["ref_energy"])) < 0.1
        # unit_test_sorf.py:101 asserts rtol = atol = 1e-4 against values printed to 5 digits;
        # the print alone rounds 5e1-sized entries by up to 5e-4, so allow 1e-3 absolute
        got = F.squeeze(0).cpu().numpy()
        assert np.abs(got - d["ref_forces"]).max() < 1e-3 + 1e-4 * np.abs(d["ref_forces"]).max()
        assert np.isclose(d["ref_forces"], got, rtol=1e-4, atol=1e-3).all()


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("case", ["benzene_c1", "aspirin_c2", "ragged_c3", "flexible_c4"])
def test_sorf_energy_and_forces_vs_oracle(case, fused):
    cfg = {
        "benzene_c1": (helpers.benzene_batch(5, 0), [1, 6], 64, 8),
        "aspirin_c2": (helpers.fixed_composition_batch(helpers.ASPIRIN, 4, 1), [1, 6, 8], 128, 16),
        "ragged_c3": (helpers.ragged_batch(9, 2), [1, 6, 7, 8, 9], 128, 4),
        # the shape of the 32768-feature configuration: four species, 27 atoms, 256 components
        "flexible_c4": (helpers.fixed_composition_batch(helpers.C12H12N2O, 2, 3, sigma=0.15), [1, 6, 7, 8], 256, 4),
    }[case]
    (coords, charges), species, npcas, nstacks = cfg
    m, (red, D, bias, alpha) = build_sorf_model(species, npcas, nstacks, fused=fused)
    prm = oracle_prm(species)
    X, Z, aid, mid, nat = make_batch(coords, charges)
    E, F, Zf = omodel.sorf_energy_forces(X, Z, aid, mid, nat, prm, species, red, D, bias, alpha, 2.0)
    gX, gZ, gaid, gmid, gnat = inputs(X, Z, aid, mid, nat)
    e, f = m.predict_opt(gX, gZ, gaid, gmid, gnat)
    close(e, E, REL_EF, "energies")
    close(f, F, REL_EF, "forces")
    for mm in range(len(nat)):
        assert (f[mm, nat[mm]:] == 0).all()
    e_only = m.predict_opt(gX.detach().clone(), gZ, gaid, gmid, gnat, forces=False)
    close(e_only, E, REL_EF, "energies, no forces")
    # the differentiable route (what a TorchScript caller runs): forward + autograd
    gX2 = gX.detach().clone().requires_grad_(True)
    e2 = m.forward(gX2, gZ, gaid, gmid, gnat)
    f2, = torch.autograd.grad(-e2.sum(), gX2)
    close(e2, E, REL_EF, "energies, autograd route")
    close(f2, F, REL_EF, "forces, autograd route")


def test_periodic_cell_energy_and_forces_both_routes():
    """Minimum-image neighbours through the whole model: `predict_opt` (no autograd graph) and
    `forward` + autograd against the oracle."""
    species = [1, 8]
    rng = np.random.default_rng(8)
    cellm = np.array([[5.0, 0.0, 0.0], [0.5, 5.2, 0.0], [0.2, 0.3, 4.9]]).T.astype(np.float32).astype(np.float64)
    inv = np.linalg.inv(cellm).astype(np.float32).astype(np.float64)
    coords = [helpers.random_geometry(rng, 6, 4.8, 1.2), helpers.random_geometry(rng, 5, 4.8, 1.2)]
    charges = [np.array([8, 1, 1, 8, 1, 1]), np.array([8, 1, 1, 1, 8])]
    X, Z, aid, mid, nat = make_batch(coords, charges)
    cell, icell = np.stack([cellm, cellm]), np.stack([inv, inv])
    m, (red, D, bias, alpha) = build_sorf_model(species, 64, 4, rcut=2.4, nRs2=10, nRs3=8)
    prm = oracle_prm(species, rcut=2.4, nRs2=10, nRs3=8)
    E, F, _ = omodel.sorf_energy_forces(X, Z, aid, mid, nat, prm, species, red, D, bias, alpha, 2.0, cell=cell,
                                        inv_cell=icell)
    gX, gZ, gaid, gmid, gnat = inputs(X, Z, aid, mid, nat)
    e, f = m.predict_opt(gX, gZ, gaid, gmid, gnat, t32(cell), t32(icell))
    close(e, E, REL_EF, "periodic energies")
    close(f, F, REL_EF, "periodic forces")
    gX2 = gX.detach().clone().requires_grad_(True)
    e2 = m.forward(gX2, gZ, gaid, gmid, gnat, t32(cell), t32(icell))
    f2, = torch.autograd.grad(-e2.sum(), gX2)
    close(e2, E, REL_EF, "periodic energies, autograd route")
    close(f2, F, REL_EF, "periodic forces, autograd route")


def test_forward_routes_agree_under_autograd():
    """forward + autograd.grad through the one-operator chain, the same chain operator by operator,
    and the reference's two-operator route: same energies, same gradients for a weighted sum of the
    energies (the upstream gradient differs per molecule), also for a single unbatched molecule."""
    species = [1, 6, 8]
    coords, charges = helpers.ragged_batch(5, 4)
    species = [1, 6, 7, 8, 9]
    X, Z, aid, mid, nat = make_batch(coords, charges)
    prm = oracle_prm(species)
    w = torch.tensor([0.5, -1.0, 2.0, 0.0, 1.5], device=dev())
    results = []
    for kw in (dict(fused=True), dict(fused=True, separate_ops=True), dict(fused=False)):
        sep = kw.pop("separate_ops", False)
        m, (red, D, bias, alpha) = build_sorf_model(species, 32, 4, **kw)
        m.separate_ops = sep
        gX, gZ, gaid, gmid, gnat = inputs(X, Z, aid, mid, nat)
        gX.requires_grad_(True)
        e = m.forward(gX, gZ, gaid, gmid, gnat)
        g, = torch.autograd.grad((e * w).sum(), gX)
        results.append((e.detach(), g))
        with torch.no_grad():                                  # no gradient asked: energies only
            e_ng = m.forward(gX.detach(), gZ, gaid, gmid, gnat)
        assert torch.equal(e_ng, e.detach())
    E, F, _ = omodel.sorf_energy_forces(X, Z, aid, mid, nat, prm, species, red, D, bias, alpha, 2.0)
    for e, g in results:
        close(e, E, REL_EF, "energies")
        close(g, -F * w.cpu().numpy()[:, None, None], REL_EF, "weighted gradient")
    # one molecule handed over unbatched: X [n,3], Z [n]
    m, _ = build_sorf_model(species, 32, 4)
    n0 = int(nat[0])
    x1 = t32(X[0, :n0]).requires_grad_(True)
    e1 = m.forward(x1, t32(Z[0, :n0]), ti32(aid[:n0]), ti32(mid[:n0]), ti32(nat[:1]))
    g1, = torch.autograd.grad(e1.sum(), x1)
    assert g1.shape == x1.shape
    close(e1, E[:1], REL_EF, "unbatched energy")
    close(g1, -F[0, :n0], REL_EF, "unbatched gradient")


def test_two_transforms_and_torch_ops_directly():
    """ntransforms = 2 through the registered operators, autograd included."""
    species = [1, 6]
    (coords, charges) = helpers.benzene_batch(2, 3)
    m, (red, D, bias, alpha) = build_sorf_model(species, 32, 4, ntransforms=2, fused=False)
    prm = oracle_prm(species)
    X, Z, aid, mid, nat = make_batch(coords, charges)
    E, F, _ = omodel.sorf_energy_forces(X, Z, aid, mid, nat, prm, species, red, D, bias, alpha, 2.0)
    e, f = m.predict_opt(*inputs(X, Z, aid, mid, nat))
    close(e, E, REL_EF)
    close(f, F, REL_EF)
    m2, _ = build_sorf_model(species, 32, 4, ntransforms=2, fused=True)
    e2, f2 = m2.predict_opt(*inputs(X, Z, aid, mid, nat))
    close(e2, E, REL_EF)
    close(f2, F, REL_EF)


def test_torchscript_roundtrip(tmp_path):
    species = [1, 6, 8]
    (coords, charges) = helpers.fixed_composition_batch(helpers.ASPIRIN, 3, 1)
    X, Z, aid, mid, nat = make_batch(coords, charges)
    for fused in (True, False):
        m, _ = build_sorf_model(species, 64, 8, fused=fused)
        gX, gZ, gaid, gmid, gnat = inputs(X, Z, aid, mid, nat)
        e0, f0 = m.predict_opt(gX, gZ, gaid, gmid, gnat)
        path = os.path.join(tmp_path, "model_%d.pt" % fused)
        m.save_jit_model(path)
        loaded = torch.jit.load(path)
        gX2 = gX.detach().clone().requires_grad_(True)
        e1 = loaded.forward(gX2, gZ, gaid, gmid, gnat)
        f1, = torch.autograd.grad(-e1.sum(), gX2)
        close(e1, e0.detach().cpu().numpy(), 1e-6, "scripted energies")
        close(f1, f0.cpu().numpy(), 1e-5, "scripted forces")
        code = loaded.code
        assert ("sorf_energy" in code) == fused
        assert ("get_SORF_coefficients" in code) == (not fused)


def test_known_answer_through_a_model_file_read_as_data(kat, tmp_path):
    """The aspirin model written in the reference's file layout (the reference's operator
    sequence, its attribute names and dtypes: checked on the host in test_model_files.py), read
    back by `from_reference_file` without unpickling, then run through the fused route, the
    reference route and `torch.jit.load` of the same file: the three agree and reproduce the
    reference's printed energy and forces (unit_test_sorf.py:59-80,93-101)."""
    from qml_lightning_amd.models.hadamard_features import HadamardFeaturesModel
    from qml_lightning_amd.representations.FCHL import FCHLCuda
    from qml_lightning_amd.utils import model_files
    d = kat
    rep = FCHLCuda(species=np.array([1, 6, 8]), rcut=6.0, nRs2=24, nRs3=22, eta2=0.28, eta3=3.2,
                   two_body_decay=2.3, three_body_weight=18.8, three_body_decay=0.65)
    rep.three_body_weight = torch.tensor(float(d["three_body_weight"]))
    src = HadamardFeaturesModel(rep=rep, elements=np.array([1, 6, 8]), ntransforms=1, sigma=2.0, llambda=1e-5,
                                npcas=128, nstacks=128, nbatch_test=256, fused=False)
    src.reductors, src.Dmat, src.bias = t32(d["reductors"]), t32(d["Dmat"].astype(np.float32)), t32(d["bias"])
    src.alpha = torch.tensor(d["alpha"], device=dev())
    src.self_energy = torch.tensor(d["self_energy"])
    src.set_subtract_self_energies(True)
    src.is_trained = True
    path = os.path.join(tmp_path, "model_sorf.pt")
    src.save_jit_model(path)
    model_files.check_reference_loadable(path)
    n = d["coordinates"].shape[0]
    Z = t32(d["charges"]).unsqueeze(0)
    ids = (torch.arange(n, dtype=torch.int32, device=dev()), torch.zeros(n, dtype=torch.int32, device=dev()), ti32([n]))
    results = []
    for fused in (True, False, None):
        m = torch.jit.load(path) if fused is None else HadamardFeaturesModel.from_reference_file(path, fused=fused)
        X = t32(d["coordinates"]).unsqueeze(0).requires_grad_(True)
        E = m.forward(X, Z, *ids)
        F, = torch.autograd.grad(-E.sum(), X)
        se = d["self_energy"] if fused is None else m.self_energy.numpy()
        total = se[d["charges"]].sum() + E.item()
        assert np.isclose(float(d["ref_energy"]), total) and abs(total - float(d["ref_energy"])) < 0.1
        got = F.squeeze(0).cpu().numpy()
        assert np.isclose(d["ref_forces"], got, rtol=1e-4, atol=1e-3).all()
        results.append((E.item(), got))
    # the reference route from the file read as data IS the scripted file's arithmetic (the forces
    # go through the FCHL19 backward kernel, whose cross-atom sums are fp32 atomics in any order)
    assert results[1][0] == results[2][0]
    assert np.abs(results[1][1] - results[2][1]).max() < 2e-6 * np.abs(results[2][1]).max()
    assert abs(results[0][0] - results[1][0]) < 1e-4 * abs(results[1][0])
    assert np.abs(results[0][1] - results[1][1]).max() < 1e-4 * np.abs(results[1][1]).max()


def test_predict_from_lists_and_predict_cuda():
    species = [1, 6, 7, 8, 9]
    coords, charges = helpers.ragged_batch(11, 4)
    m, (red, D, bias, alpha) = build_sorf_model(species, 64, 4)
    prm = oracle_prm(species)
    c32 = [np.asarray(c, dtype=np.float32) for c in coords]
    X, Z, aid, mid, nat = make_batch(coords, charges)
    E, F, _ = omodel.sorf_energy_forces(X, Z, aid, mid, nat, prm, species, red, D, bias, alpha, 2.0)
    nmax = int(nat.max())
    e, f = m.predict(c32, charges, nmax, forces=True)          # one batch: the fused route widens nbatch_test
    close(e, E, REL_EF, "predict energies")
    close(f, F, REL_EF, "predict forces")
    assert m._fused_batch(nmax) == m.fused_batch_atoms // nmax
    m.fused_batch_atoms = 0                                    # batches of nbatch_test = 5 molecules: 5 + 5 + 1
    assert m._fused_batch(nmax) == 5
    e, f = m.predict(c32, charges, nmax, forces=True)
    close(e, E, REL_EF, "predict energies, three batches")
    close(f, F, REL_EF, "predict forces, three batches")
    # the explicit-Jacobian route (fp64 rows times alpha) gives the same numbers
    e2, f2 = m.predict_cuda(c32, charges, nmax, forces=True, print_info=False)
    close(e2, E, REL_EF, "predict_cuda energies")
    close(f2, F, REL_EF, "predict_cuda forces")


@pytest.mark.parametrize("mode", ["EF", "E", "F"])
def test_training_rows_and_gram_vs_oracle(mode):
    species = [1, 6]
    coords, charges = helpers.benzene_batch(6, 0)
    m, (red, D, bias, alpha) = build_sorf_model(species, 16, 4)
    prm = oracle_prm(species)
    rng = np.random.default_rng(14)
    E = rng.normal(size=6) if "E" in mode else None
    Fo = [rng.normal(size=(12, 3)) for _ in range(6)] if "F" in mode else None
    c32 = [np.asarray(c, dtype=np.float32) for c in coords]
    rows, ys = [], []
    for i in range(0, 6, 4):          # nbatch_train = 4
        X, Z, aid, mid, nat = make_batch(coords[i:i + 4], charges[i:i + 4])
        r, y = omodel.sorf_training_rows(X, Z, aid, mid, nat, prm, species, red, D, bias, 2.0,
                                         E=E[i:i + 4] if E is not None else None,
                                         F=np.array(Fo[i:i + 4]) if Fo is not None else None)
        rows.append(r)
        ys.append(y)
    R, Y = np.concatenate(rows), np.concatenate(ys)
    ZTZ_ref, ZTy_ref = osorf.gram(R, Y)
    ZTZ, ZTy = m.build_Z_components(c32, charges, E=E, F=Fo, print_info=False)
    close(ZTZ, ZTZ_ref, 2e-5, "ZTZ " + mode)      # products of 1e-5-accurate features
    close(ZTy, ZTy_ref, 2e-5, "ZTy " + mode)
    for kw in (dict(ntiles=3), dict(cpu_solve=True), dict(use_specialized_matmul=True),
               dict(ntiles=2, use_specialized_matmul=True)):
        a, b = m.build_Z_components(c32, charges, E=E, F=Fo, print_info=False, **kw)
        close(a, ZTZ_ref, 2e-5, "ZTZ %s %s" % (mode, kw))
        close(b, ZTy_ref, 2e-5, "ZTy %s %s" % (mode, kw))
    if mode == "EF":
        # rows of one batch, and the train/predict loop closing on itself
        data = m.format_data(c32[:4], charges[:4], E=E[:4], F=Fo[:4])
        close(m._batch_rows(data, True), rows[0], REL_REP, "rows")
        m.train(c32, charges, E=E, F=Fo, print_info=False)
        assert m.alpha.shape == (m.nfeatures(),) and torch.isfinite(m.alpha).all()


def test_training_rows_of_a_padded_array_batch_vs_oracle_and_list_route():
    """A ragged training batch handed over as one zero-padded array pair with E [B] and F [B,n,3]
    (device-side formatter, element index by a device sort) gives the rows of the fp64 oracle and,
    bit for bit, the rows and Z^T Z of the per-molecule-list route (kernel.py:601-722,143-160)."""
    species = [1, 6, 7, 8, 9]
    coords, charges = helpers.ragged_batch(9, 4)
    m, (red, D, bias, alpha) = build_sorf_model(species, 64, 2)
    m.nbatch_train = 9
    prm = oracle_prm(species)
    rng = np.random.default_rng(3)
    c32 = [np.asarray(c, dtype=np.float32) for c in coords]
    B, n = len(c32), max(len(q) for q in charges)
    E = rng.normal(size=B)
    Fl = [rng.normal(size=(len(q), 3)) for q in charges]
    Xp, Qp, Fp = np.zeros((B, n, 3), dtype=np.float32), np.zeros((B, n), dtype=np.float32), np.zeros((B, n, 3))
    for i, (c, q, f) in enumerate(zip(c32, charges, Fl)):
        Xp[i, :len(q)], Qp[i, :len(q)], Fp[i, :len(q)] = c, q, f
    dl = m.format_data(c32, charges, E=E, F=Fl)
    dp = m.format_data(Xp, Qp, E=E, F=Fp)
    for key in ("coordinates", "charges", "natom_counts", "atomIDs", "molIDs", "energies", "forces"):
        assert dl[key].dtype == dp[key].dtype and torch.equal(dl[key], dp[key]), key
    rl, rp = m._batch_rows(dl, True), m._batch_rows(dp, True)
    assert torch.equal(rl, rp)
    X, Z, aid, mid, nat = make_batch(coords, charges)
    Fo = np.zeros((B, n, 3))
    for i, f in enumerate(Fl):
        Fo[i, :len(f)] = f
    r, y = omodel.sorf_training_rows(X, Z, aid, mid, nat, prm, species, red, D, bias, 2.0, E=E, F=Fo)
    close(rp, r, REL_REP, "rows of the padded batch")
    close(m._targets(dp, B, True, True), y, 1e-14, "targets of the padded batch")
    # the element index of the device sort is the molecule-major search of the reference
    types = m._sort_species_tensor()
    assert [float(v) for v in types.cpu()] == [float(e) for e in species]
    Zl, yl = m.build_Z_components(c32, charges, E=E, F=Fl, print_info=False)
    Zp, yp = m.build_Z_components(Xp, Qp, E=E, F=Fp, print_info=False)
    assert torch.equal(Zl, Zp) and torch.allclose(yl, yp, rtol=1e-12, atol=1e-12)   # Z^T y: fp64 atomics
    # a model whose elements are a permuted subset of the batch's: atoms of other elements give no rows
    from qml_lightning_amd.models.hadamard_features import HadamardFeaturesModel
    sub = HadamardFeaturesModel(rep=m.rep, elements=np.array([8, 1, 6]), ntransforms=1, sigma=2.0, npcas=64, nstacks=2)
    perm = [species.index(e) for e in (8, 1, 6)]
    sub.reductors, sub.Dmat, sub.bias = m.reductors[perm].clone(), m.Dmat[perm].clone(), m.bias[perm].clone()
    ds = sub.format_data(Xp, Qp, E=E, F=Fp)
    rs = sub._batch_rows(ds, True)
    # the oracle's element loop (hadamard_features.py:99) never selects the N and F atoms either
    r_sub, _ = omodel.sorf_training_rows(X, Z, aid, mid, nat, prm, [8, 1, 6], red[perm], D[perm], bias[perm], 2.0,
                                         E=E, F=Fo)
    close(rs, r_sub, REL_REP, "rows of a model with fewer elements than the batch")


@pytest.mark.parametrize("ragged", [False, True])
def test_format_data_of_padded_arrays_equals_the_list_route(ragged):
    """One zero-padded array pair goes through the device-side formatter; lists of per-molecule
    arrays through the host one (kernel.py:601-722).  Same tensors, same predictions."""
    species = [1, 6, 8]
    coords, charges = helpers.fixed_composition_batch(helpers.ASPIRIN, 5, 1)
    if ragged:
        keep = [21, 9, 15, 21, 4]
        coords = [c[:k] for c, k in zip(coords, keep)]
        charges = [q[:k] for q, k in zip(charges, keep)]
    m, _ = build_sorf_model(species, 32, 4)
    c32 = [np.asarray(c, dtype=np.float32) for c in coords]
    n = max(len(q) for q in charges)
    Xp = np.zeros((len(c32), n, 3), dtype=np.float32)
    Qp = np.zeros((len(c32), n), dtype=np.float32)
    for i, (c, q) in enumerate(zip(c32, charges)):
        Xp[i, :len(q)] = c
        Qp[i, :len(q)] = q
    a = m.format_data(c32, charges)
    b = m.format_data(Xp, Qp)
    for key in ("coordinates", "charges", "natom_counts", "atomIDs", "molIDs"):
        assert a[key].dtype == b[key].dtype and torch.equal(a[key], b[key]), key
    if not ragged:
        # lists of equal-size molecules are stacked and take the device formatter too; the same molecules
        # followed by a smaller one take the host formatter: the same tensors for the molecules they share
        g = m.format_data(c32 + [c32[0][:4]], list(charges) + [charges[0][:4]])
        natoms = sum(len(q) for q in charges)
        assert torch.equal(g["coordinates"][:len(c32)], a["coordinates"]) and torch.equal(g["charges"][:len(c32)], a["charges"])
        assert torch.equal(g["natom_counts"][:len(c32)], a["natom_counts"])
        assert torch.equal(g["atomIDs"][:natoms], a["atomIDs"]) and torch.equal(g["molIDs"][:natoms], a["molIDs"])
    ea, fa = m.predict(c32, charges, n, forces=True, print_info=False)
    eb, fb = m.predict(Xp, Qp, n, forces=True, print_info=False)
    assert torch.equal(ea, eb)
    assert (fa - fb).abs().max() <= 1e-6 * fa.abs().max()   # the force sums use float atomics: order varies
    bad = Qp.copy()
    bad[0, 0] = 0.0                                      # a hole before real atoms
    with pytest.raises(RuntimeError):
        m.format_data(Xp, bad)


def test_kernels_follow_the_current_stream():
    """Every launch goes to torch's current stream: the same step issued inside a side-stream
    context (after that stream has been made to wait for the inputs) gives the same numbers, and
    nothing is left running on the default stream."""
    species = [1, 6, 8]
    coords, charges = helpers.fixed_composition_batch(helpers.ASPIRIN, 6, 1)
    m, _ = build_sorf_model(species, 64, 8)
    X, Z, aid, mid, nat = make_batch(coords, charges)
    args = inputs(X, Z, aid, mid, nat)
    e0, f0 = m.energies_and_forces(*args)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        e1, f1 = m.energies_and_forces(*args)
        done = torch.cuda.Event()
        done.record(side)
    done.synchronize()
    assert torch.equal(e0, e1)
    assert (f0 - f1).abs().max() <= 1e-6 * f0.abs().max()


@pytest.mark.parametrize("kind", ["sorf", "rff"])
def test_predict_step_replayed_from_a_captured_graph(kind):
    """The predict step allocates only through torch and records no memset nodes, so it can be captured
    in a HIP graph.  The graph is replayed five times with changed coordinates, with the program's own
    eager work and synchronisations between the replays, and every replay is checked against the eager
    result of the same coordinates (SORF energies bit-equal: they are summed in a fixed order; the RFF
    kernel adds its feature shares with fp32 atomics; forces to the rounding of the atomic scatters)."""
    species = [1, 6, 8]
    coords, charges = helpers.fixed_composition_batch(helpers.ASPIRIN, 3, 1)
    if kind == "sorf":
        m, _ = build_sorf_model(species, 128, 8)
    else:
        from qml_lightning_amd.models.random_features import RandomFourrierFeaturesModel
        from qml_lightning_amd.representations.FCHL import FCHLCuda
        rep = FCHLCuda(species=np.array(species))
        np.random.seed(3)
        m = RandomFourrierFeaturesModel(rep=rep, elements=np.array(species), sigma=3.0, llambda=1e-5, npcas=64,
                                        nstacks=4, nbatch_train=4, nbatch_test=5)
        red, _, _, alpha = helpers.model_weights(len(species), rep.get_repsize(), 64, 4)
        m.reductors = t32(red)
        m.alpha = torch.tensor(alpha, device=dev())
        m.is_trained = True
    X, Z, aid, mid, nat = inputs(*make_batch(coords, charges))
    Xs = X.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            m.energies_and_forces(Xs, Z, aid, mid, nat)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        eg, fg = m.energies_and_forces(Xs, Z, aid, mid, nat)
    for it in range(5):
        Xp = X + 0.02 * it
        ee, fe = m.energies_and_forces(Xp, Z, aid, mid, nat)      # eager work between the replays
        torch.cuda.synchronize()
        Xs.copy_(Xp)
        graph.replay()
        torch.cuda.synchronize()
        if kind == "sorf":
            assert torch.equal(eg, ee), (kind, it)
        else:
            assert (eg - ee).abs().max() <= 1e-6 * ee.abs().max(), (kind, it)
        assert (fg - fe).abs().max() <= 1e-5 * fe.abs().max(), (kind, it)
    assert not torch.equal(fe, m.energies_and_forces(X, Z, aid, mid, nat)[1])   # the inputs did change the result


def test_reductor_fit_matches_an_svd_of_the_samples():
    """get_reductors (kernel.py:447-540): per element the leading left singular vectors of the
    sampled representations; here via the Gram matrix and an eigensolve, checked against numpy's SVD."""
    from qml_lightning_amd.models.kernel import BaseKernel
    rng = np.random.default_rng(2)
    mat = (rng.normal(size=(700, 60)) * np.logspace(0, -3, 60)).astype(np.float32)
    U, S = BaseKernel._left_singular_vectors(torch.tensor(mat, device=dev()))
    Un, Sn, _ = np.linalg.svd(mat.astype(np.float64).T, full_matrices=False)
    assert U.shape == (60, 60) and U.dtype == torch.float32
    close(S, Sn, 1e-5, "singular values")
    Ud = U.double().cpu().numpy()
    for k in (1, 8, 32):                                   # same leading subspaces
        assert np.abs(Ud[:, :k] @ Ud[:, :k].T - Un[:, :k] @ Un[:, :k].T).max() < 1e-5
    assert np.abs(Ud.T @ Ud - np.eye(60)).max() < 1e-5
    assert (Ud[np.abs(Ud).argmax(axis=0), np.arange(60)] > 0).all()     # the sign convention

    species = [1, 6, 8]
    coords, charges = helpers.fixed_composition_batch(helpers.ASPIRIN, 12, 1)
    c32 = [np.asarray(c, dtype=np.float32) for c in coords]
    m, _ = build_sorf_model(species, 32, 4)
    m.reductors = torch.zeros_like(m.reductors)
    np.random.seed(0)
    torch.manual_seed(0)
    m.get_reductors(c32, charges, npcas=32, print_info=False)
    first = m.reductors.clone()
    for e in range(3):
        P = first[e].double()
        assert (P.T @ P - torch.eye(32, dtype=torch.float64, device=dev())).abs().max() < 1e-5
    np.random.seed(0)
    torch.manual_seed(0)
    m.get_reductors(c32, charges, npcas=32, print_info=False)
    assert torch.equal(first, m.reductors)                  # seeded selection, deterministic vectors
    with pytest.raises(RuntimeError):                       # 4 oxygens x 2 molecules < 32 components
        m.get_reductors(c32[:2], charges[:2], npcas=32, print_info=False)


def test_grid_search_shares_the_gram_matrix_across_lambdas():
    """hyperparam_opt_nested_cv (kernel.py:249-347) builds the representation, its Jacobian and the
    projected rows once per fold, the features and Z^T Z once per (sigma, fold); every grid point
    must score exactly as a fresh train() + predict() at that point does."""
    species = [1, 6]
    coords, charges = helpers.benzene_batch(8, 3)
    c32 = [np.asarray(c, dtype=np.float32) for c in coords]
    rng = np.random.default_rng(21)
    E = rng.normal(size=8)
    Fo = [rng.normal(size=(12, 3)) for _ in range(8)]
    sigmas, lambdas, kfolds = [2.0, 3.0, 4.5], [1e-3, 1e-1], 2
    m, _ = build_sorf_model(species, 16, 4)
    jacobian_calls = []
    real_jacobian = m.rep.get_representation_and_derivative
    m.rep.get_representation_and_derivative = lambda *a, **k: (jacobian_calls.append(1), real_jacobian(*a, **k))[1]
    printed = []
    import builtins
    real_print = builtins.print
    builtins.print = lambda *a, **k: printed.append(a)
    try:
        best = m.hyperparam_opt_nested_cv(c32, charges, E, Fo, sigmas=sigmas, lambdas=lambdas, kfolds=kfolds)
    finally:
        builtins.print = real_print
    got = {(a[1], a[3]): a[5] for a in printed if a and a[0] == "sigma"}
    # 4 training molecules per fold = one batch of nbatch_train = 4: one Jacobian launch per fold,
    # whatever the number of sigmas and lambdas
    assert len(jacobian_calls) == kfolds
    from sklearn.model_selection import KFold
    expect = {}
    for sg in sigmas:
        for lm in lambdas:
            m2, _ = build_sorf_model(species, 16, 4, sigma=sg)
            m2.llambda = lm
            tot = 0.0
            for tr, te in KFold(n_splits=kfolds, shuffle=False).split(c32):
                pick = lambda seq, ids: [seq[i] for i in ids]
                m2.train(pick(c32, tr), pick(charges, tr), pick(E, tr), pick(Fo, tr), print_info=False)
                ep, fp = m2.predict(pick(c32, te), pick(charges, te), 12, forces=True, print_info=False)
                et = torch.tensor(np.array(pick(E, te)), device=dev())
                ft = torch.tensor(np.array(pick(Fo, te)), device=dev())
                tot += 0.5 * float(torch.mean(torch.abs(ep - et)) + torch.mean(torch.abs(fp - ft)))
            expect[(sg, lm)] = tot / kfolds
    assert set(got) == set(expect)
    for k in expect:      # two builds of Z^T Z differ in summation order; the solve amplifies that
        assert abs(got[k] - expect[k]) <= 1e-6 * max(1.0, abs(expect[k])), (k, got[k], expect[k])
    assert best == min(expect, key=expect.get)
    # without room for the cache the search falls back to one full build per (sigma, fold): same scores
    m3, _ = build_sorf_model(species, 16, 4)
    m3.grid_search_cache_bytes = 0
    printed.clear()
    builtins.print = lambda *a, **k: printed.append(a)
    try:
        best3 = m3.hyperparam_opt_nested_cv(c32, charges, E, Fo, sigmas=sigmas, lambdas=lambdas, kfolds=kfolds)
    finally:
        builtins.print = real_print
    got3 = {(a[1], a[3]): a[5] for a in printed if a and a[0] == "sigma"}
    for k in expect:
        assert abs(got3[k] - expect[k]) <= 1e-6 * max(1.0, abs(expect[k])), (k, got3[k], expect[k])
    assert best3 == best


def test_rff_model_vs_oracle():
    from qml_lightning_amd.models.random_features import RandomFourrierFeaturesModel
    from qml_lightning_amd.representations.FCHL import FCHLCuda
    species = [1, 6, 8]
    coords, charges = helpers.fixed_composition_batch(helpers.ASPIRIN, 3, 1)
    rep = FCHLCuda(species=np.array(species))
    np.random.seed(5)
    m = RandomFourrierFeaturesModel(rep=rep, elements=np.array(species), sigma=2.0, nstacks=4, npcas=32,
                                    nbatch_train=2, nbatch_test=2)
    red, _, _, _ = helpers.model_weights(3, rep.get_repsize(), 32, 4)
    m.reductors = t32(red)
    rng = np.random.default_rng(13)
    alpha = rng.normal(size=m.nfeatures())
    m.alpha = torch.tensor(alpha, device=dev())
    m.is_trained = True
    W = m.W.double().cpu().numpy()
    b = m.b.double().cpu().numpy()
    prm = oracle_prm(species)
    X, Z, aid, mid, nat = make_batch(coords, charges)
    E, F, Zf = omodel.rff_energy_forces(X, Z, aid, mid, nat, prm, species, red, W, b,
                                        alpha.astype(np.float32).astype(np.float64))
    e, f = m.predict_opt(*inputs(X, Z, aid, mid, nat))
    close(e, E, REL_EF, "rff energies")
    close(f, F, REL_EF, "rff forces")
    # training rows (fp64 kernels) against the oracle's rows
    c32 = [np.asarray(c, dtype=np.float32) for c in coords]
    data = m.format_data(c32, charges)
    rows = m._batch_rows(data, True)
    rep_o, J, _ = omodel.representation(X, Z, aid, mid, nat, prm, jacobian=True)
    G = np.zeros((3, 21, 3, m.nfeatures()))
    Zc = np.zeros((3, m.nfeatures()))
    for ei, el in enumerate(species):
        mask = Z.astype(int) == el
        idx = np.nonzero(mask)[0]
        sub = osorf.project(rep_o[mask], red[ei])
        Zc += osorf.rff_features(sub, W[ei], b[ei], idx, 3)
        G += osorf.rff_derivative_features(sub, osorf.project(J[mask], red[ei]), W[ei], b[ei], idx, 3)
    close(rows[:3], Zc, REL_REP, "rff Z rows")
    close(rows[3:], G.reshape(-1, m.nfeatures()), REL_REP, "rff G rows")
    s = torch.jit.script(m)
    gX = t32(X).requires_grad_(True)
    e2 = s.forward(gX, t32(Z), ti32(aid), ti32(mid), ti32(nat))
    close(e2, E, REL_EF, "scripted rff energies")


@pytest.mark.parametrize("npcas,nstacks,case", [(64, 3, "aspirin"), (128, 2, "ragged")])
def test_rff_fused_forward_vs_oracle(npcas, nstacks, case):
    """The single-kernel RFF predict path (energies, autograd forces, energies only, TorchScript)."""
    from qml_lightning_amd.models.random_features import RandomFourrierFeaturesModel
    from qml_lightning_amd.representations.FCHL import FCHLCuda
    if case == "aspirin":
        species = [1, 6, 8]
        coords, charges = helpers.fixed_composition_batch(helpers.ASPIRIN, 7, 1)
    else:
        species = [1, 6, 7, 8, 9]
        coords, charges = helpers.ragged_batch(11, 2)
    rep = FCHLCuda(species=np.array(species))
    np.random.seed(6)
    m = RandomFourrierFeaturesModel(rep=rep, elements=np.array(species), sigma=2.0, nstacks=nstacks, npcas=npcas)
    assert m.fused
    red, _, _, _ = helpers.model_weights(len(species), rep.get_repsize(), npcas, nstacks)
    m.reductors = t32(red)
    alpha = np.random.default_rng(14).normal(size=m.nfeatures())
    m.alpha = torch.tensor(alpha, device=dev())
    m.is_trained = True
    prm = oracle_prm(species)
    X, Z, aid, mid, nat = make_batch(coords, charges)
    E, F, _ = omodel.rff_energy_forces(X, Z, aid, mid, nat, prm, species, red, m.W.double().cpu().numpy(),
                                       m.b.double().cpu().numpy(), alpha.astype(np.float32).astype(np.float64))
    e, f = m.predict_opt(*inputs(X, Z, aid, mid, nat))
    close(e, E, REL_EF, "fused rff energies")
    close(f, F, REL_EF, "fused rff forces")
    e_only = m.predict_opt(*inputs(X, Z, aid, mid, nat), forces=False)
    close(e_only, E, REL_EF, "fused rff energies, no forces")
    s = torch.jit.script(m)
    gX = t32(X).requires_grad_(True)
    e2 = s.forward(gX, t32(Z), ti32(aid), ti32(mid), ti32(nat))
    f2, = torch.autograd.grad(-e2.sum(), gX)
    close(e2, E, REL_EF, "scripted fused rff energies")
    close(f2, F, REL_EF, "scripted fused rff forces")
    # the same chain operator by operator
    m.separate_ops = True
    gX3 = t32(X).requires_grad_(True)
    e3 = m.forward(gX3, t32(Z), ti32(aid), ti32(mid), ti32(nat))
    f3, = torch.autograd.grad(-e3.sum(), gX3)
    close(e3, E, REL_EF, "rff energies, separate operators")
    close(f3, F, REL_EF, "rff forces, separate operators")


def test_fd_helper_matches_jacobian():
    """FCHLCuda.rep_deriv_fd, the reference's own check of its analytic Jacobian
    (unit_tests/representation/test_fchl_derivative.py:60-82)."""
    from qml_lightning_amd.representations.FCHL import FCHLCuda
    coords, charges = helpers.benzene_batch(1, 2)
    rep = FCHLCuda(species=np.array([1, 6]), nRs2=8, nRs3=6)
    X, Z, aid, mid, nat = make_batch(coords, charges)
    gX, gZ, gaid, gmid, gnat = inputs(X, Z, aid, mid, nat)
    r, J = rep.get_representation_and_derivative(gX, gZ, gaid, gmid, gnat)
    fd = rep.rep_deriv_fd(gX, gZ, gaid, gmid, gnat, dx=0.005)
    # fp32 finite differences: the reference only prints this norm; 2 % of the scale is
    # what fp32 cancellation at dx = 0.005 allows
    assert (fd - J.double()).abs().max() < 0.02 * J.abs().max()


def test_scripted_model_runs_in_a_host_without_python(tmp_path):
    """tests/cpp/run_scripted (libtorch only) loads libqmll_torch.so, a model file saved here and
    a batch, and must print the energies and forces this process computes."""
    import subprocess
    from qml_lightning_amd import ops
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "tests", "cpp", "run_scripted")
    if ops.OPS_BACKEND != "c++" or not os.path.exists(exe):
        pytest.skip("needs libqmll_torch.so and tests/cpp/run_scripted (python -m qml_lightning_amd.build)")
    species = [1, 6, 8]
    (coords, charges) = helpers.fixed_composition_batch(helpers.ASPIRIN, 3, 1)
    X, Z, aid, mid, nat = make_batch(coords, charges)
    gX, gZ, gaid, gmid, gnat = inputs(X, Z, aid, mid, nat)

    class Batch(torch.nn.Module):
        def __init__(self):
            super().__init__()
            for name, t in (("X", gX), ("Z", gZ), ("atomIDs", gaid), ("molIDs", gmid), ("atom_counts", gnat)):
                self.register_buffer(name, t.detach().clone())

        def forward(self):
            return self.X

    batch_path = os.path.join(tmp_path, "batch.pt")
    torch.jit.script(Batch()).save(batch_path)
    for fused in (True, False):
        m, _ = build_sorf_model(species, 64, 8, fused=fused)
        e0, f0 = m.predict_opt(gX.detach().clone(), gZ, gaid, gmid, gnat)
        path = os.path.join(tmp_path, "model_%d.pt" % fused)
        m.save_jit_model(path)
        torch.cuda.synchronize()
        res = subprocess.run([exe, ops.TORCH_LIB_PATH, path, batch_path], capture_output=True, text=True, timeout=300)
        assert res.returncode == 0, res.stderr[-2000:]
        lines = res.stdout.split()
        ne = int(lines[1])
        e = np.array(lines[2:2 + ne], dtype=np.float64)
        nf = int(lines[3 + ne])
        f = np.array(lines[4 + ne:4 + ne + nf], dtype=np.float64).reshape(f0.shape)
        close(e, e0.detach().cpu().numpy(), 1e-6, "energies from the C++ host")
        close(f, f0.cpu().numpy(), 1e-5, "forces from the C++ host")


@pytest.mark.parametrize("nmol,npcas,nstacks", [(12, 16, 4), (4, 64, 8)])
def test_training_at_the_default_regularisation_vs_fp64_oracle_rows(nmol, npcas, nstacks):
    """train() at the shipped default lambda = 1e-11 (hadamard_features.py:16): alpha solved from the
    library's rows (force-feature rows summed over a molecule's atoms in fp32 before they are widened;
    the reference widens every product, cuda/hadamard_kernel.cu:710) against alpha solved in numpy from
    the fp64 oracle rows.  Both the overdetermined case (444 rows, 64 features) and the underdetermined
    one (148 rows, 512 features: Z^T Z + lambda I has a condition number near 1 / eps).  alpha itself is
    not comparable there (the normal matrix amplifies rounding by its condition number); what a user
    sees is: the fit reproduces its training targets equally well, and held-out molecules are predicted
    alike, to well below the fit's own error."""
    species = [1, 6]
    coords, charges = helpers.benzene_batch(nmol + 3, 5)
    m, (red, D, bias, _) = build_sorf_model(species, npcas, nstacks)
    m.llambda = 1e-11
    m.nbatch_train = 5
    prm = oracle_prm(species)
    rng = np.random.default_rng(3)
    c32 = [np.asarray(c, dtype=np.float32) for c in coords]
    # smooth targets: a fixed random model's own energies and forces plus a little noise
    _, _, _, a_true = helpers.model_weights(2, prm.repsize, npcas, nstacks, 1, 77)
    X, Z, aid, mid, nat = make_batch(coords, charges)
    E_all, F_all, _ = omodel.sorf_energy_forces(X, Z, aid, mid, nat, prm, species, red, D, bias, 0.05 * a_true, 2.0)
    E_all = E_all + 1e-3 * rng.normal(size=E_all.shape)
    F_all = F_all + 1e-3 * rng.normal(size=F_all.shape)
    tr, te = slice(0, nmol), slice(nmol, nmol + 3)
    m.train(c32[tr], charges[tr], E=list(E_all[tr]), F=[f for f in F_all[tr]], print_info=False)
    rows, y = omodel.sorf_training_rows(*make_batch(coords[tr], charges[tr]), prm, species, red, D, bias, 2.0,
                                        E=E_all[tr], F=F_all[tr])
    ZTZ, ZTy = osorf.gram(rows, y)
    a_ref = osorf.regularised_solve(ZTZ, ZTy, 1e-11)[:, 0]
    a_gpu = m.alpha.double().cpu().numpy()
    # the fit on its own training rows (fp64 rows of the oracle, both alphas)
    res_gpu = np.abs(rows @ a_gpu - y[:, 0]).max()
    res_ref = np.abs(rows @ a_ref - y[:, 0]).max()
    scale = np.abs(y).max()
    print("default lambda, %d rows x %d features: training residual gpu %.2e, oracle %.2e (targets up to %.2e)"
          % (rows.shape[0], rows.shape[1], res_gpu, res_ref, scale))
    assert res_gpu <= max(3.0 * res_ref, 2e-4 * scale)
    # held-out molecules through the fp64 oracle with either alpha, and through the library's predict
    Xt, Zt, at, mt, nt = make_batch(coords[te], charges[te])
    E_ref, F_ref, _ = omodel.sorf_energy_forces(Xt, Zt, at, mt, nt, prm, species, red, D, bias, a_ref, 2.0)
    E_g, F_g, _ = omodel.sorf_energy_forces(Xt, Zt, at, mt, nt, prm, species, red, D, bias, a_gpu, 2.0)
    e_dev = np.abs(E_g - E_ref).max() / np.abs(E_ref).max()
    f_dev = np.abs(F_g - F_ref).max() / np.abs(F_ref).max()
    # the yardstick: the same solve from the oracle's rows with noise of 1e-7 of their largest entry, a
    # hundredth of the parity tolerance of the features and the size of fp32 rounding in a feature
    # value (the reference computes every feature value in fp32 too, cuda/hadamard_kernel.cu:561,583)
    noisy = rows + 1e-7 * np.abs(rows).max() * np.random.default_rng(9).normal(size=rows.shape)
    a_n = osorf.regularised_solve(*osorf.gram(noisy, y), 1e-11)[:, 0]
    E_p, F_p, _ = omodel.sorf_energy_forces(Xt, Zt, at, mt, nt, prm, species, red, D, bias, a_n, 2.0)
    e_yard = np.abs(E_p - E_ref).max() / np.abs(E_ref).max()
    f_yard = np.abs(F_p - F_ref).max() / np.abs(F_ref).max()
    print("held-out predictions vs the fp64-trained alpha: library-trained energies %.2e forces %.2e; "
          "oracle rows with 1e-7 noise: energies %.2e forces %.2e" % (e_dev, f_dev, e_yard, f_yard))
    assert e_dev <= max(1e-3, 3.0 * e_yard) and f_dev <= max(1e-3, 3.0 * f_yard)
    # and the rows themselves: the force-feature rows (fp32 sum over a molecule's atoms) are as close to
    # the fp64 oracle as the energy rows (every value widened before it is added)
    if nmol <= 5:                      # one batch of nbatch_train = 5 molecules holds them all
        data = m.format_data(c32[tr], charges[tr], E=list(E_all[tr]), F=[f for f in F_all[tr]])
        got = m._batch_rows(data, True).cpu().numpy()
        err = np.abs(got - rows)
        rms_e = np.sqrt((err[:nmol] ** 2).mean()) / np.abs(rows[:nmol]).max()
        rms_f = np.sqrt((err[nmol:] ** 2).mean()) / np.abs(rows[nmol:]).max()
        print("rows vs oracle, rms error over largest entry: energy rows %.2e, force rows %.2e" % (rms_e, rms_f))
        assert rms_f <= max(2.0 * rms_e, 1e-7) and rms_e <= 5e-7
    e, f = m.predict(c32[te], charges[te], 12, forces=True, print_info=False)
    close(e, E_g, 5e-4, "library predict with its own alpha, energies")     # fp32 contraction with an alpha of large entries
    close(f, F_g, 5e-4, "library predict with its own alpha, forces")


@pytest.mark.parametrize("kind", ["sorf", "rff"])
def test_forces_operator_equals_minus_the_gradient_of_the_energy_operator(kind):
    """energies_and_forces takes energies and forces from ONE operator that builds no autograd graph and
    applies the sign inside its last kernel (qmll_fchl19_vjp_scaled): same energies as `forward`, forces
    equal to minus autograd's gradient, for a padded ragged batch and for a single unbatched molecule; with
    a coordinate tensor that requires a gradient it refuses instead of returning something detached."""
    species = [1, 6, 7, 8, 9]
    coords, charges = helpers.ragged_batch(7, 11)
    m = (build_sorf_model(species, 32, 4)[0] if kind == "sorf" else build_rff_model(species, 64, 4)[0])
    X, Z, aid, mid, nat = make_batch(coords, charges)
    gX, gZ, gaid, gmid, gnat = inputs(X, Z, aid, mid, nat)
    e, f = m.energies_and_forces(gX, gZ, gaid, gmid, gnat)
    Xg = gX.clone().requires_grad_(True)
    e2 = m.forward(Xg, gZ, gaid, gmid, gnat)
    g, = torch.autograd.grad(e2.sum(), Xg)
    etol = 2e-6 * float(e.abs().max())          # the RFF kernel adds its feature shares with fp32 atomics
    assert (e - e2.detach()).abs().max() <= (0.0 if kind == "sorf" else etol)
    assert (f + g).abs().max() <= 2e-6 * g.abs().max()            # the cross-atom sums use atomics
    e_only, none = m.energies_and_forces(gX, gZ, gaid, gmid, gnat, forces=False)
    assert none is None and (e_only - e).abs().max() <= (0.0 if kind == "sorf" else etol)
    op = torch.ops.qml_lightning_sorf.fchl_sorf_forces if kind == "sorf" else torch.ops.qml_lightning_sorf.fchl_rff_forces
    rep = m.rep
    head = (gZ, rep.species, gaid, gmid, gnat, torch.empty(0, 3, 3, device=dev()), torch.empty(0, 3, 3, device=dev()), rep.Rs2,
            rep.Rs3, rep.eta2, rep.eta3, rep.two_body_decay, rep.three_body_weight, rep.three_body_decay, rep.rcut)
    if kind == "sorf":
        tail = (m.reductors, m.Dmat, m.bias, m.alpha.float(), torch.tensor(float(np.sqrt(np.float32(m.npcas)) / m.sigma)),
                m.ntransforms, m.sort_species)
    else:
        tail = (m.reductors, m.W, m.b, m.alpha.float(), m.sort_species)
    with pytest.raises(RuntimeError, match="no autograd graph"):
        op(Xg, *head, *tail)
    # one unbatched molecule: [n,3] coordinates and [n] charges in, [n,3] forces out
    n0 = int(gnat[0])
    one = op(gX[0], gZ[0], rep.species, gaid[:n0], gmid[:n0], gnat[:1], *head[5:], *tail)
    assert one[1].shape == gX[0].shape
    assert (one[1] - f[0]).abs().max() <= 2e-6 * f.abs().max() and abs(float(one[0][0] - e[0])) <= 1e-5 * float(e.abs().max())
