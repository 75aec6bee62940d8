"""Shared synthetic inputs for the parity tests (seeded, deterministic)."""
from oracle import fchl19
from qml_lightning_amd.utils.synthetic import (ASPIRIN, C12H12N2O, benzene_batch,  # noqa: F401
                                               fixed_composition_batch, model_weights, ragged_batch,
                                               random_geometry)


def kat_params(d):
    return fchl19.FCHLParams(d["species"], rcut=float(d["rcut"]), eta2=float(d["eta2"]), eta3=float(d["eta3"]),
                             two_body_decay=float(d["two_body_decay"]),
                             raw_three_body_weight=float(d["three_body_weight"]),
                             three_body_decay=float(d["three_body_decay"]), Rs2=d["Rs2"], Rs3=d["Rs3"])
