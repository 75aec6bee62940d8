"""The oracle against the reference's own known-answer vector
(unit_tests/models/unit_test_sorf.py with the weights of saved_models/model_sorf.pt,
committed as tests/golden/aspirin_sorf_kat.npz)."""
import numpy as np

from oracle import model
from tests import helpers


def test_oracle_reproduces_reference_energy_and_forces(kat):
    d = kat
    prm = helpers.kat_params(d)
    # the reference feeds fp32 coordinates (unit_test_sorf.py:82)
    xyz = d["coordinates"].astype(np.float32).astype(np.float64)
    X, Z, aid, mid, nat = model.format_batch([xyz], [d["charges"]])
    E, F, _ = model.sorf_energy_forces(X, Z, aid, mid, nat, prm, d["elements"], d["reductors"],
                                       d["Dmat"].astype(np.float64), d["bias"], d["alpha"], float(d["sigma"]))
    total = E[0] + d["self_energy"][d["charges"]].sum()
    # reference assertion (unit_test_sorf.py:100): np.isclose(ref_energy, total); the printed
    # value is an fp32 number near 4e5 (spacing 0.03)
    assert np.isclose(float(d["ref_energy"]), total)
    assert abs(total - float(d["ref_energy"])) < 0.04
    # reference assertion (unit_test_sorf.py:101): rtol = atol = 1e-4; ref_forces are printed
    # to 5 significant figures, which alone allows 5e-4 on the 5e1-sized entries
    assert np.isclose(d["ref_forces"], F[0], rtol=1e-4, atol=1e-4).all()
    assert np.abs(F[0] - d["ref_forces"]).max() < 1e-3


def test_reductors_are_orthonormal_and_D_is_sign(kat):
    U = kat["reductors"].astype(np.float64)
    for e in range(3):
        assert np.abs(U[e].T @ U[e] - np.eye(128)).max() < 5e-3
    assert set(np.unique(kat["Dmat"])) == {-1, 1}
    assert kat["bias"].min() >= 0 and kat["bias"].max() <= 2 * np.pi + 1e-6
