"""Every registered operator and every function of the pybind-named modules, called once with
the reference's positional argument order and checked against the oracle: the operators of
qml_lightning/cuda/torchscript/FCHL19.cpp:318-333 and the modules fchl_gpu
(cuda/fchl_cuda.cpp:204-212), pairlist_gpu (cuda/pairlist_cuda.cpp:67-72), rff_gpu
(cuda/random_features.cpp:35-39).  Also: a model whose element list differs from the
representation's species list, the Python operator registrations run in a child process,
and host-side refusals of tables that do not fit each other."""
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from oracle import fchl19
from oracle import model as omodel
from oracle import sorf as osorf
from tests import helpers
from tests.test_gpu_kernels import REL_EF, REL_REP, close, dev, make_batch, oracle_prm, t32, ti32
from tests.test_gpu_model import build_sorf_model, inputs

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _case():
    """Ragged batch (padding in every molecule but the largest), five species."""
    coords, charges = helpers.ragged_batch(5, 6)
    species = [1, 6, 7, 8, 9]
    prm = oracle_prm(species, nRs2=9, nRs3=7)
    X, Z, aid, mid, nat = make_batch(coords, charges)
    cnt, nl = fchl19.neighbours(X, nat, prm.rcut)
    ty = fchl19.element_types(Z, nat, prm.species)
    return prm, X, Z, aid, mid, nat, cnt, nl, ty


def _scalars(prm):
    return (torch.tensor(prm.eta2), torch.tensor(prm.eta3), torch.tensor(prm.two_body_decay),
            torch.tensor(prm.three_body_weight), torch.tensor(prm.three_body_decay), torch.tensor(prm.rcut))


def test_fchl_operators_of_the_torchscript_library_vs_oracle():
    """torch.ops.qml_lightning_fchl.{get_num_neighbours, get_neighbour_list, get_element_types,
    get_fchl_and_derivative (gradients False and True), fchl_forwards, fchl_backwards}."""
    import qml_lightning_amd  # noqa: F401
    prm, X, Z, aid, mid, nat, cnt, nl, ty = _case()
    O = torch.ops.qml_lightning_fchl
    empty = torch.empty(0, 3, 3, device=dev())
    gX, gZ, gaid, gmid, gnat = inputs(X, Z, aid, mid, nat)
    rcut = torch.tensor(prm.rcut)
    g_cnt = O.get_num_neighbours(gX, gnat, rcut, empty, empty)
    assert g_cnt.dtype == torch.int32 and (g_cnt.cpu().numpy() == cnt).all()
    g_nl = O.get_neighbour_list(gX, gnat, g_cnt.max(), rcut, empty, empty)
    assert g_nl.dtype == torch.int32 and (g_nl.cpu().numpy() == nl).all()
    g_ty = O.get_element_types(gX, gZ, gnat, t32(prm.species))
    assert g_ty.dtype == torch.int32 and (g_ty.cpu().numpy() == ty).all()

    rep = fchl19.forward(X, ty, aid, mid, nl, cnt, prm)
    J = fchl19.jacobian(X, ty, aid, mid, nl, cnt, prm)
    args = (gX, gZ, t32(prm.species), gaid, gmid, gnat, empty, empty, t32(prm.Rs2), t32(prm.Rs3)) + _scalars(prm)
    out = O.get_fchl_and_derivative(*args, False)
    assert len(out) == 1
    close(out[0], rep, REL_REP, "get_fchl_and_derivative(False)")
    out = O.get_fchl_and_derivative(*args, True)
    assert len(out) == 2 and out[1].shape == (len(nat), X.shape[1], X.shape[1], 3, prm.repsize)
    close(out[0], rep, REL_REP, "get_fchl_and_derivative(True) rep")
    close(out[1], J, REL_REP, "get_fchl_and_derivative(True) jacobian")
    for m in range(len(nat)):                      # rows and columns of padded slots stay zero
        assert (out[1][m, nat[m]:] == 0).all() and (out[1][m, :, nat[m]:] == 0).all()
    close(O.fchl_forwards(*args), rep, REL_REP, "fchl_forwards")
    g = np.random.default_rng(3).normal(size=rep.shape)
    close(O.fchl_backwards(t32(g), *args), np.einsum("mif,mijxf->mjx", g, J), REL_EF, "fchl_backwards")


def test_fchl_gpu_module_with_the_reference_argument_order():
    """fchl_gpu.{get_element_types_gpu, get_fchl_representation, get_fchl_derivative,
    get_fchl_and_derivative, fchl_backwards} and pairlist_gpu.*: 18 / 19 positional arguments
    as in cuda/fchl_cuda.cpp:64-202, scalars as Python floats; with the lists of pairlist_gpu
    and without a list (the kernel then finds the neighbours itself, from the atom counts the
    charges give)."""
    from qml_lightning_amd.cuda import fchl_gpu, pairlist_gpu
    prm, X, Z, aid, mid, nat, cnt, nl, ty = _case()
    gX, gZ, gaid, gmid, gnat = inputs(X, Z, aid, mid, nat)
    species = t32(prm.species)
    g_cnt = pairlist_gpu.get_num_neighbours_gpu(gX, gnat, prm.rcut)
    g_nl = pairlist_gpu.get_neighbour_list_gpu(gX, gnat, int(g_cnt.max().item()), prm.rcut)
    assert (g_cnt.cpu().numpy() == cnt).all() and (g_nl.cpu().numpy() == nl).all()
    filled = g_nl.clone()
    pairlist_gpu.safe_fill_gpu(filled)              # pairlist_cuda.cpp:39-45: fill with -1 in place
    assert filled.data_ptr() != g_nl.data_ptr() and (filled == -1).all()
    g_ty = fchl_gpu.get_element_types_gpu(gX, gZ, gnat, species)
    assert (g_ty.cpu().numpy() == ty).all()

    rep = fchl19.forward(X, ty, aid, mid, nl, cnt, prm)
    J = fchl19.jacobian(X, ty, aid, mid, nl, cnt, prm)
    g = np.random.default_rng(4).normal(size=rep.shape)
    v = np.einsum("mif,mijxf->mjx", g, J)
    empty = torch.empty(0, 3, 3, device=dev())
    tail = (t32(prm.Rs2), t32(prm.Rs3), prm.eta2, prm.eta3, prm.two_body_decay, prm.three_body_weight,
            prm.three_body_decay, prm.rcut)
    for lists in ((g_nl, g_cnt), (None, None)):
        head = (gX, gZ, species, g_ty, empty, empty, gaid, gmid) + lists
        what = "with lists" if lists[0] is not None else "no lists"
        close(fchl_gpu.get_fchl_representation(*head, *tail), rep, REL_REP, "get_fchl_representation " + what)
        close(fchl_gpu.get_fchl_derivative(*head, *tail), J, REL_REP, "get_fchl_derivative " + what)
        out = fchl_gpu.get_fchl_and_derivative(*head, *tail, True)
        close(out[0], rep, REL_REP, "get_fchl_and_derivative rep " + what)
        close(out[1], J, REL_REP, "get_fchl_and_derivative jacobian " + what)
        out = fchl_gpu.get_fchl_and_derivative(*head, *tail, False)
        assert len(out) == 1
        close(out[0], rep, REL_REP, "get_fchl_and_derivative(False) " + what)
        close(fchl_gpu.fchl_backwards(*head, *tail, t32(g)), v, REL_EF, "fchl_backwards " + what)


def test_rff_gpu_module_vs_oracle():
    """rff_gpu.get_rff and get_rff_derivatives (cuda/random_features.cpp:11-33): accumulate in
    place into fp64 tensors; atoms in arbitrary molecule order (the atomics route)."""
    from qml_lightning_amd.cuda import rff_gpu
    rng = np.random.default_rng(9)
    A, n, d, F, nmol = 37, 5, 32, 96, 6
    x = rng.normal(size=(A, d)).astype(np.float32)
    grad = rng.normal(size=(A, n, 3, d)).astype(np.float32)
    W = rng.normal(size=(d, F)) / 8.0
    b = rng.uniform(0, 2 * np.pi, F)
    order = rng.integers(0, nmol, A).astype(np.int32)
    start = rng.normal(size=(nmol, F))
    Zf = torch.tensor(start, device=dev())
    rff_gpu.get_rff(t32(x), torch.tensor(W, device=dev()), torch.tensor(b, device=dev()), ti32(order), Zf)
    close(Zf, start + osorf.rff_features(x, W, b, order, nmol), 1e-12, "get_rff")
    gstart = rng.normal(size=(nmol, n, 3, F))
    G = torch.tensor(gstart, device=dev())
    rff_gpu.get_rff_derivatives(t32(x), t32(grad), torch.tensor(W, device=dev()), torch.tensor(b, device=dev()),
                                ti32(order), G)
    close(G, gstart + osorf.rff_derivative_features(x, grad, W, b, order, nmol), 1e-12, "get_rff_derivatives")


@pytest.mark.parametrize("elements", [[1, 6, 8], [8, 1, 7, 6], [6, 9, 1, 8, 7]])
def test_model_elements_that_differ_from_the_representation_species(elements):
    """The representation knows H, C, N, O, F; the model a subset of them (atoms of the other
    elements shape their neighbours' representations but carry no energy of their own, as with
    the reference's `Z == e` masks over the model's elements, models/hadamard_features.py:99-107)
    or the same elements in another order.  All three SORF routes and the RFF model."""
    from qml_lightning_amd.models.hadamard_features import HadamardFeaturesModel
    from qml_lightning_amd.models.random_features import RandomFourrierFeaturesModel
    from qml_lightning_amd.representations.FCHL import FCHLCuda
    rep_species = [1, 6, 7, 8, 9]
    coords, charges = helpers.ragged_batch(5, 6)
    assert {int(q) for qs in charges for q in qs} == set(rep_species)     # every element occurs
    X, Z, aid, mid, nat = make_batch(coords, charges)
    prm = oracle_prm(rep_species, nRs2=10, nRs3=8)
    npcas, nstacks = 64, 4
    red, D, bias, alpha = helpers.model_weights(len(elements), prm.repsize, npcas, nstacks, 1, 31)
    alpha64 = alpha.astype(np.float32).astype(np.float64)
    E, F, _ = omodel.sorf_energy_forces(X, Z, aid, mid, nat, prm, elements, red, D.astype(np.float64), bias, alpha64, 2.0)
    for kw in (dict(fused=True), dict(fused=True, separate_ops=True), dict(fused=False)):
        rep = FCHLCuda(species=np.array(rep_species), nRs2=10, nRs3=8)
        m = HadamardFeaturesModel(rep=rep, elements=np.array(elements), ntransforms=1, sigma=2.0, npcas=npcas,
                                  nstacks=nstacks, **kw)
        m.reductors, m.Dmat, m.bias = t32(red), t32(D), t32(bias)
        m.alpha = torch.tensor(alpha, device=dev())
        m.is_trained = True
        gX, gZ, gaid, gmid, gnat = inputs(X, Z, aid, mid, nat)
        gX.requires_grad_(True)
        e = m.forward(gX, gZ, gaid, gmid, gnat)
        f, = torch.autograd.grad(-e.sum(), gX)
        close(e, E, REL_EF, "energies %s" % kw)
        close(f, F, REL_EF, "forces %s" % kw)
        if kw == dict(fused=True):
            e2, f2 = m.predict_opt(gX.detach().clone(), gZ, gaid, gmid, gnat)
            close(e2, E, REL_EF, "predict_opt energies")
            close(f2, F, REL_EF, "predict_opt forces")
            s = torch.jit.script(m)                 # the scripted model carries its own element list
            close(s.forward(gX.detach(), gZ, gaid, gmid, gnat), E, REL_EF, "scripted energies")
    # training rows use the model's elements too: G.alpha must equal the forces above
    data = m.format_data([np.asarray(c, dtype=np.float32) for c in coords], charges, E=list(E), F=[f_[:k] for f_, k in zip(F, nat)])
    rows = m._batch_rows(data, True)
    out = rows @ torch.tensor(alpha64, device=dev())
    close(out[:len(nat)], E, REL_EF, "rows . alpha, energies")
    close(out[len(nat):].reshape(F.shape), F, REL_EF, "rows . alpha, forces")

    np.random.seed(8)
    rep = FCHLCuda(species=np.array(rep_species), nRs2=10, nRs3=8)
    r = RandomFourrierFeaturesModel(rep=rep, elements=np.array(elements), sigma=2.0, nstacks=3, npcas=npcas)
    assert r.fused
    r.reductors = t32(red)
    ralpha = np.random.default_rng(5).normal(size=r.nfeatures())
    r.alpha = torch.tensor(ralpha, device=dev())
    r.is_trained = True
    E, F, _ = omodel.rff_energy_forces(X, Z, aid, mid, nat, prm, elements, red, r.W.double().cpu().numpy(),
                                       r.b.double().cpu().numpy(), ralpha.astype(np.float32).astype(np.float64))
    e, f = r.predict_opt(*inputs(X, Z, aid, mid, nat))
    close(e, E, REL_EF, "rff energies")
    close(f, F, REL_EF, "rff forces")


def test_chain_operator_refuses_a_model_that_does_not_fit_the_representation():
    m, _ = build_sorf_model([1, 6, 8], 64, 4)
    coords, charges = helpers.fixed_composition_batch(helpers.ASPIRIN, 2, 1)
    args = inputs(*make_batch(coords, charges))
    good = m.reductors
    m.reductors = good[:2].contiguous()                 # two reductors, three species, no model species given
    with pytest.raises(RuntimeError, match="model"):
        m.energies_and_forces(*args)
    m.reductors = good[:, :100].contiguous()            # representation length
    with pytest.raises(RuntimeError, match="reductors"):
        m.energies_and_forces(*args)
    m.reductors = good
    m.alpha = m.alpha[:100]                             # alpha from another feature count
    with pytest.raises(RuntimeError, match="alpha"):
        m.energies_and_forces(*args)


def test_tables_that_do_not_fit_each_other_are_refused_before_any_launch():
    """Diagonals, bias, alpha, W taken from another npcas / nstacks must raise, not read out of bounds."""
    from qml_lightning_amd import ops
    x = torch.zeros(4, 64, device=dev())
    D = torch.ones(1, 2, 64, device=dev())
    bias, alpha = torch.zeros(128, device=dev()), torch.zeros(128, device=dev())
    idx = ti32([0, 0, 1, 1])
    with pytest.raises(RuntimeError, match="last dimensions"):
        ops.sorf_forward(x, torch.ones(1, 2, 32, device=dev()), 1.0, 1)
    with pytest.raises(RuntimeError, match="last dimensions"):
        torch.ops.qml_lightning_sorf.get_SORF_coefficients(x, torch.ones(1, 2, 32, device=dev()), torch.tensor(1.0),
                                                           torch.tensor(1))
    with pytest.raises(RuntimeError, match="diagonals"):
        ops.sorf_adjoint(torch.zeros(4, 2, 64, device=dev()), torch.ones(1, 3, 64, device=dev()), 1.0, 1)
    c = torch.zeros(4, 128, device=dev())
    with pytest.raises(RuntimeError, match="bias"):
        ops.cos_features(c, bias[:64], 2, idx)
    with pytest.raises(RuntimeError, match="bias"):
        torch.ops.qml_lightning_sorf.get_cos_features(c, bias[:64], torch.tensor(2), idx)
    with pytest.raises(RuntimeError, match="bias"):
        ops.cos_features_backward(torch.zeros(2, 128, device=dev()), c, bias[:64], 2, idx)
    with pytest.raises(RuntimeError, match="bias"):
        ops.sin_coeffs(c, bias[:64], torch.zeros(4, 128, dtype=torch.float64, device=dev()))
    e = torch.zeros(4, device=dev())
    with pytest.raises(RuntimeError, match="do not fit"):
        ops.sorf_energy_fused(x, D, bias, alpha[:64], None, 1.0, 1, e)
    with pytest.raises(RuntimeError, match="do not fit"):
        ops.sorf_energy_fused(x, D, bias[:64], alpha, None, 1.0, 1, e)
    off, ss = ti32([0, 4]), ti32([0, 1, 2, 3])
    Dm = D[None]
    with pytest.raises(RuntimeError, match="do not fit"):
        ops.sorf_energy_sorted(x, off, ss, Dm, bias[None, :64], alpha, 1.0, 1, 4)
    with pytest.raises(RuntimeError, match="do not fit"):
        ops.sorf_energy_sorted(x, off, ss, Dm, bias[None], alpha[:3], 1.0, 1, 4)
    with pytest.raises(RuntimeError, match="do not fit"):
        torch.ops.qml_lightning_sorf.sorf_energy_sorted(x, off, ss, Dm, bias[None], alpha[:3], torch.tensor(1.0),
                                                        torch.tensor(1), 4, False)
    W, b = torch.zeros(1, 64, 96, device=dev()), torch.zeros(1, 96, device=dev())
    with pytest.raises(RuntimeError, match="alpha"):
        ops.rff_energy_sorted(x, off, ss, W, b, alpha[:32], 4)
    with pytest.raises(RuntimeError, match="alpha"):
        torch.ops.qml_lightning_sorf.rff_energy_sorted(x, off, ss, W, b, alpha[:32], 4, False)
    with pytest.raises(RuntimeError, match="do not fit"):
        ops.rff_features(x, torch.zeros(32, 96, dtype=torch.float64, device=dev()),
                         torch.zeros(96, dtype=torch.float64, device=dev()), idx,
                         torch.zeros(2, 96, dtype=torch.float64, device=dev()))


def test_known_answer_vector_through_the_python_operator_registrations():
    """The torch.library definitions in ops.py / models/hadamard_features.py (what serves when
    libqmll_torch.so is not there) in a fresh process: the reference's aspirin known-answer
    vector, both routes, and autograd through the one-operator chain."""
    code = r'''
import os, sys
import numpy as np, torch
sys.path.insert(0, %r)
import qml_lightning_amd
from qml_lightning_amd import ops
assert ops.OPS_BACKEND == "python", ops.OPS_BACKEND
from qml_lightning_amd.models.hadamard_features import HadamardFeaturesModel
from qml_lightning_amd.representations.FCHL import FCHLCuda
d = np.load(os.path.join(%r, "tests", "golden", "aspirin_sorf_kat.npz"))
dev = torch.device("cuda:0")
t32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.float32, device=dev)
for fused, sep in ((True, False), (True, True), (False, False)):
    rep = FCHLCuda(species=np.array([1, 6, 8]), rcut=6.0, nRs2=24, nRs3=22, eta2=0.28, eta3=3.2,
                   two_body_decay=2.3, three_body_weight=18.8, three_body_decay=0.65)
    rep.three_body_weight = torch.tensor(float(d["three_body_weight"]))
    m = HadamardFeaturesModel(rep=rep, elements=np.array([1, 6, 8]), ntransforms=1, sigma=2.0, llambda=1e-5,
                              npcas=128, nstacks=128, fused=fused, separate_ops=sep)
    m.reductors, m.Dmat, m.bias = t32(d["reductors"]), t32(d["Dmat"].astype(np.float32)), t32(d["bias"])
    m.alpha = torch.tensor(d["alpha"], device=dev)
    n = d["coordinates"].shape[0]
    X = t32(d["coordinates"]).unsqueeze(0).requires_grad_(True)
    Z = t32(d["charges"]).unsqueeze(0)
    E = m.forward(X, Z, torch.arange(n, dtype=torch.int32, device=dev), torch.zeros(n, dtype=torch.int32, device=dev),
                  torch.tensor([n], dtype=torch.int32, device=dev))
    F, = torch.autograd.grad(-E.sum(), X)
    total = d["self_energy"][d["charges"]].sum() + E.item()
    assert abs(total - float(d["ref_energy"])) < 0.1, total
    got = F.squeeze(0).cpu().numpy()
    assert np.isclose(d["ref_forces"], got, rtol=1e-4, atol=1e-3).all(), np.abs(got - d["ref_forces"]).max()
    if fused and not sep:
        s = torch.jit.script(m)
        assert abs(float(s.forward(X.detach(), Z, torch.arange(n, dtype=torch.int32, device=dev),
                                   torch.zeros(n, dtype=torch.int32, device=dev),
                                   torch.tensor([n], dtype=torch.int32, device=dev))) - E.item()) < 1e-3
print("python-ops-ok")
''' % (ROOT, ROOT)
    env = dict(os.environ, QML_LIGHTNING_AMD_PY_OPS="1")
    res = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=600, env=env)
    assert res.returncode == 0 and "python-ops-ok" in res.stdout, (res.stdout[-1500:], res.stderr[-3000:])
