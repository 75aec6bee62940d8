"""Model files both ways, on the host: the weights-only reader against the reference-held
`model_sorf.pt` (where the reference tree exists) and the committed fixture made from it,
`from_reference_file`, and the operator schema / attribute layout of files saved here
against what the reference's own files carry (hadamard_features.py:253-255,
torchscript/FCHL19.cpp:318-333, torchscript/SORF.cpp:138-150)."""
import io
import os
import pickle
import zipfile

import numpy as np
import pytest
import torch

from qml_lightning_amd.utils import model_files

REF_FILE = "/root/reference/unit_tests/models/saved_models/model_sorf.pt"
needs_reference = pytest.mark.skipif(not os.path.exists(REF_FILE), reason="the reference tree is not on this machine")

# attribute -> (dtype, ndim) of the tensors a reference-saved SORF model carries, as its own file
# records them (read once from REF_FILE; the table is data, kept here so the layout check also
# runs where the reference tree is absent)
REFERENCE_LAYOUT = {
    "elements": ("int64", 1), "reductors": ("float32", 3), "element2index": ("int64", 1),
    "ntransforms": ("int64", 0), "species": ("float32", 1), "Dmat": ("float32", 4), "bias": ("float32", 2),
    "alpha": ("float64", 1),
}
REFERENCE_REP_LAYOUT = {
    "species": ("float32", 1), "rcut": ("float32", 0), "nRs2": ("int64", 0), "nRs3": ("int64", 0),
    "eta2": ("float32", 0), "eta3": ("float32", 0), "two_body_decay": ("float32", 0),
    "three_body_weight": ("float32", 0), "three_body_decay": ("float32", 0), "Rs2": ("float32", 1),
    "Rs3": ("float32", 1), "pi": ("float32", 1),
}
REFERENCE_SCALARS = {"npcas": int, "sigma": float, "llambda": float, "nstacks": int, "nbatch_train": int,
                     "nbatch_test": int, "is_trained": bool, "hartree2kcalmol": float,
                     "_convert_from_hartree_to_kcal": bool, "_subtract_self_energies": bool}


def _small_model(fused, trained=True):
    from qml_lightning_amd.models.hadamard_features import HadamardFeaturesModel
    from qml_lightning_amd.representations.FCHL import FCHLCuda
    np.random.seed(5)
    rep = FCHLCuda(species=np.array([1, 6, 8]), nRs2=6, nRs3=4, eta3=3.2, three_body_weight=18.8)
    m = HadamardFeaturesModel(rep=rep, elements=np.array([1, 6, 8]), ntransforms=2, sigma=2.5, llambda=1e-7, npcas=16,
                              nstacks=3, nbatch_test=17, fused=fused)
    g = torch.Generator().manual_seed(3)
    m.reductors = torch.randn(m.reductors.shape, generator=g).to(m.device)
    if trained:
        m.alpha = torch.randn(m.nfeatures(), generator=g, dtype=torch.float64).to(m.device)
        m.is_trained = True
    m.self_energy = torch.tensor([0.0, -0.5, 0, 0, 0, 0, -37.8, 0, -75.0], dtype=torch.float64)
    m.set_subtract_self_energies(True)
    return m


def _layout(tree, table):
    return {k: (str(np.asarray(tree[k]).dtype), np.asarray(tree[k]).ndim) for k in table}


@needs_reference
def test_reader_reproduces_the_fixture_from_the_reference_held_file(kat):
    tree = model_files.read_attribute_tree(REF_FILE)
    assert tree["__class__"] == "__torch__.qml_lightning.models.hadamard_features.HadamardFeaturesModel"
    for k in ("self_energy", "elements", "reductors", "element2index", "ntransforms", "bias", "alpha"):
        assert np.array_equal(tree[k], kat[k]) and tree[k].dtype == kat[k].dtype, k
    assert np.array_equal(tree["Dmat"], kat["Dmat"].astype(np.float32))
    for k in ("species", "rcut", "eta2", "eta3", "two_body_decay", "three_body_weight", "three_body_decay", "Rs2",
              "Rs3"):
        assert np.array_equal(tree["rep"][k], kat[k]), k
    assert (tree["sigma"], tree["npcas"], tree["nstacks"]) == (float(kat["sigma"]), int(kat["npcas"]),
                                                                int(kat["nstacks"]))
    # the layout table of this file is the reference's
    assert _layout(tree, REFERENCE_LAYOUT) == REFERENCE_LAYOUT
    assert _layout(tree["rep"], REFERENCE_REP_LAYOUT) == REFERENCE_REP_LAYOUT
    for k, t in REFERENCE_SCALARS.items():
        assert type(tree[k]) is t, k
    assert model_files.archive_version(REF_FILE) == 4
    # and the operators its code calls are the three the reference's forward uses, positional
    assert model_files.check_reference_loadable(REF_FILE) == {
        "qml_lightning_fchl::fchl_forwards": 1, "qml_lightning_sorf::get_SORF_coefficients": 1,
        "qml_lightning_sorf::get_cos_features": 1}


REF_FILE_2 = "/root/reference/examples/MD17/model_sorf.pt"


@pytest.mark.skipif(not os.path.exists(REF_FILE_2), reason="the reference checkout is not here")
def test_reader_on_the_references_second_model_file():
    """examples/MD17/model_sorf.pt: other weights, no expected outputs with it; the reader finds the same
    layout, operators and hyper-parameters, orthonormal reductor columns and +-1 diagonals, and
    from_reference_file builds a trained model from it."""
    tree = model_files.read_attribute_tree(REF_FILE_2)
    assert tree["__class__"] == "__torch__.qml_lightning.models.hadamard_features.HadamardFeaturesModel"
    assert _layout(tree, REFERENCE_LAYOUT) == REFERENCE_LAYOUT
    assert _layout(tree["rep"], REFERENCE_REP_LAYOUT) == REFERENCE_REP_LAYOUT
    for k, t in REFERENCE_SCALARS.items():
        assert type(tree[k]) is t, k
    assert set(model_files.check_reference_loadable(REF_FILE_2)) == {
        "qml_lightning_fchl::fchl_forwards", "qml_lightning_sorf::get_SORF_coefficients",
        "qml_lightning_sorf::get_cos_features"}
    ne, R, d = tree["reductors"].shape
    assert (ne, d) == (len(tree["elements"]), tree["npcas"]) and R == tree["rep"]["fp_size"]
    U = tree["reductors"].astype(np.float64)
    for e in range(ne):
        assert np.abs(U[e].T @ U[e] - np.eye(d)).max() < 5e-3
    assert set(np.unique(tree["Dmat"])) <= {-1.0, 1.0}
    assert tree["Dmat"].shape == (ne, int(tree["ntransforms"]), tree["nstacks"], d)
    assert tree["bias"].shape == (ne, tree["nstacks"] * d) and 0.0 <= tree["bias"].min() and tree["bias"].max() <= 2 * np.pi
    assert tree["alpha"].shape == (tree["nstacks"] * d,) and tree["alpha"].dtype == np.float64
    from qml_lightning_amd.models.hadamard_features import HadamardFeaturesModel
    m = HadamardFeaturesModel.from_reference_file(REF_FILE_2)
    assert m.is_trained and m.nfeatures() == tree["nstacks"] * d
    assert np.array_equal(m.alpha.cpu().numpy(), tree["alpha"])


@needs_reference
def test_from_reference_file_builds_the_model_of_the_known_answer_test(kat):
    from qml_lightning_amd.models.hadamard_features import HadamardFeaturesModel
    m = HadamardFeaturesModel.from_reference_file(REF_FILE)
    assert m.is_trained and m.fused and m.subtract_self_energies() and not m.convert_hartree2kcal()
    assert (m.npcas, m.nstacks, int(m.ntransforms), m.sigma, m.llambda) == (128, 128, 1, 2.0, 1e-5)
    assert m.nbatch_test == 256 and m.nfeatures() == 16384
    for k in ("reductors", "bias", "alpha", "self_energy", "element2index", "elements"):
        got = getattr(m, k)
        assert np.array_equal(got.cpu().numpy(), kat[k]) and str(got.dtype).endswith(str(kat[k].dtype)), k
    assert np.array_equal(m.Dmat.cpu().numpy(), kat["Dmat"].astype(np.float32))
    rep = m.rep
    assert rep.fp_size == 336 and rep.nspecies == 3
    for k in ("species", "rcut", "eta2", "eta3", "two_body_decay", "three_body_weight", "three_body_decay", "Rs2",
              "Rs3"):
        got = getattr(rep, k)
        assert got.dtype == torch.float32 and np.array_equal(got.cpu().numpy(), kat[k]), k
    # scalar hyper-parameters stay 0-d host tensors (the operators read them with .item())
    assert rep.rcut.dim() == 0 and rep.rcut.device.type == "cpu"
    # the self energies of the known-answer molecule, as unit_test_sorf.py:97-100 adds them
    se = m.self_energy[torch.from_numpy(kat["charges"]).long()].sum().item()
    assert abs(se - float(kat["self_energy"][kat["charges"]].sum())) == 0.0


def test_a_file_saved_here_with_the_reference_route_has_the_references_schema_and_layout(tmp_path):
    m = _small_model(fused=False)
    path = str(tmp_path / "model_sorf.pt")
    m.save_jit_model(path)
    # only the reference's operators, with its positional all-Tensor argument lists
    calls = model_files.check_reference_loadable(path)
    assert calls == {"qml_lightning_fchl::fchl_forwards": 1, "qml_lightning_sorf::get_SORF_coefficients": 1,
                     "qml_lightning_sorf::get_cos_features": 1}
    sites = model_files.called_operators(path)
    assert sites["qml_lightning_fchl::fchl_forwards"][0][:2] == ["X", "Z"]
    tree = model_files.read_attribute_tree(path)
    # a class scripted more than once in a process gets a mangled module path: compare the class name
    assert tree["__class__"].split(".")[-1] == "HadamardFeaturesModel"
    assert tree["rep"]["__class__"].split(".")[-1] == "FCHLCuda"
    assert _layout(tree, REFERENCE_LAYOUT) == REFERENCE_LAYOUT
    assert _layout(tree["rep"], REFERENCE_REP_LAYOUT) == REFERENCE_REP_LAYOUT
    for k, t in REFERENCE_SCALARS.items():
        assert type(tree[k]) is t, k
    assert str(tree["self_energy"].dtype) == "float64"
    # the forward signature a caller of a reference-saved file relies on
    code = "\n".join(model_files.archive_code(path).values())
    assert "def forward(self" in code
    for arg in ("X: Tensor", "Z: Tensor", "atomIDs: Tensor", "molIDs: Tensor", "atom_counts: Tensor"):
        assert arg in code


def test_a_fused_file_is_recognised_as_needing_this_librarys_operators(tmp_path):
    path = str(tmp_path / "fused.pt")
    _small_model(fused=True).save_jit_model(path)
    assert "qml_lightning_sorf::fchl_sorf_energy" in model_files.called_operators(path)
    with pytest.raises(ValueError, match="do not register"):
        model_files.check_reference_loadable(path)


@pytest.mark.parametrize("fused", [False, True])
def test_round_trip_through_a_file_saved_here(tmp_path, fused):
    from qml_lightning_amd.models.hadamard_features import HadamardFeaturesModel
    m = _small_model(fused=fused)
    path = str(tmp_path / "m.pt")
    m.save_jit_model(path)
    r = HadamardFeaturesModel.from_reference_file(path, fused=not fused)
    assert r.fused is (not fused)
    for k in ("reductors", "Dmat", "bias", "alpha", "self_energy", "element2index", "elements", "species"):
        a, b = getattr(m, k), getattr(r, k)
        assert a.dtype == b.dtype and torch.equal(a.cpu(), b.cpu()), k
    for k in ("Rs2", "Rs3", "rcut", "eta2", "eta3", "two_body_decay", "three_body_weight", "three_body_decay", "nRs2",
              "nRs3", "species"):
        a, b = getattr(m.rep, k), getattr(r.rep, k)
        assert a.dtype == b.dtype and torch.equal(a.cpu(), b.cpu()), k
    assert (r.sigma, r.llambda, r.npcas, r.nstacks, int(r.ntransforms), r.nbatch_test) == (2.5, 1e-7, 16, 3, 2, 17)
    assert r.subtract_self_energies() and r.is_trained


def test_rff_round_trip(tmp_path):
    from qml_lightning_amd.models.random_features import RandomFourrierFeaturesModel
    from qml_lightning_amd.representations.FCHL import FCHLCuda
    np.random.seed(2)
    rep = FCHLCuda(species=np.array([1, 6]), nRs2=5, nRs3=3)
    m = RandomFourrierFeaturesModel(rep=rep, elements=np.array([1, 6]), sigma=1.5, nstacks=4, npcas=8, fused=False)
    m.alpha = torch.arange(m.nfeatures(), dtype=torch.float64).to(m.device)
    m.is_trained = True
    path = str(tmp_path / "model_rff.pt")
    m.save_jit_model(path)
    assert model_files.check_reference_loadable(path) == {"qml_lightning_fchl::fchl_forwards": 1}
    before = np.random.get_state()[1].copy()
    r = RandomFourrierFeaturesModel.from_reference_file(path)
    assert np.array_equal(before, np.random.get_state()[1])       # reading a file draws nothing
    for k in ("W", "b", "alpha", "reductors"):
        assert torch.equal(getattr(m, k).cpu(), getattr(r, k).cpu()), k
    assert r.nfeatures() == 32 and r.sigma == 1.5
    with pytest.raises(ValueError, match="not a HadamardFeaturesModel"):
        from qml_lightning_amd.models.hadamard_features import HadamardFeaturesModel
        HadamardFeaturesModel.from_reference_file(path)


class _Boom:
    def __reduce__(self):
        return (os.system, ("echo executed > %s" % _Boom.target,))


def test_reader_executes_nothing_and_refuses_foreign_callables(tmp_path):
    """An archive whose pickle program names a callable: unpickling would run it; the reader
    only walks the opcodes, treats the name as a label and refuses it."""
    _Boom.target = str(tmp_path / "side_effect")
    buf = io.BytesIO()
    pickle.dump({"alpha": _Boom()}, buf, protocol=2)
    path = str(tmp_path / "evil.pt")
    with zipfile.ZipFile(path, "w") as z:
        z.writestr("evil/data.pkl", buf.getvalue())
        z.writestr("evil/version", "4\n")
    with pytest.raises(ValueError, match="not one a TorchScript archive uses"):
        model_files.read_attribute_tree(path)
    assert not os.path.exists(_Boom.target)
    with pytest.raises(ValueError, match="not a TorchScript archive"):
        bad = str(tmp_path / "empty.pt")
        with zipfile.ZipFile(bad, "w") as z:
            z.writestr("readme", "x")
        model_files.read_attribute_tree(bad)


def test_strided_and_offset_tensors_are_read_as_saved(tmp_path):
    """A tensor attribute that is a view (offset, non-contiguous strides) of its storage."""
    class M(torch.nn.Module):
        def __init__(self):
            super().__init__()
            base = torch.arange(24, dtype=torch.float32).reshape(4, 6)
            self.view = base[1:, ::2].t()
            self.scalar = torch.tensor(7, dtype=torch.int64)

        def forward(self, x):
            return x + self.view.sum() + self.scalar
    path = str(tmp_path / "views.pt")
    m = M()
    torch.jit.script(m).save(path)
    tree = model_files.read_attribute_tree(path)
    assert np.array_equal(tree["view"], m.view.numpy()) and tree["view"].shape == (3, 3)
    assert tree["scalar"].shape == () and int(tree["scalar"]) == 7
