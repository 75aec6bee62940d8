"""Write tests/golden/aspirin_sorf_kat.npz from the reference's own known-answer test.

Data only: the tensors are the raw little-endian storages inside the reference's
saved model (``unit_tests/models/saved_models/model_sorf.pt``, an uncompressed zip), found
through the package's weights-only reader (``qml_lightning_amd/utils/model_files.py``: the
attribute tree of ``data.pkl`` walked opcode by opcode, storages read with
``numpy.frombuffer``); nothing from the file is unpickled, imported or executed.  Coordinates, charges and the expected energy / forces are the
literals of ``unit_tests/models/unit_test_sorf.py:11-31,57,59-80``.

Run once in the build container (the reference tree does not exist on the GPU box):
    python tests/golden/make_aspirin_fixture.py
"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
from qml_lightning_amd.utils import model_files  # noqa: E402

REF = "/root/reference/unit_tests/models/saved_models/model_sorf.pt"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "aspirin_sorf_kat.npz")

# attributes of the model and of its `rep` sub-module that the known-answer test needs
MODEL_TENSORS = ("self_energy", "elements", "reductors", "element2index", "ntransforms", "Dmat", "bias", "alpha")
REP_TENSORS = ("species", "rcut", "eta2", "eta3", "two_body_decay", "three_body_weight", "three_body_decay", "Rs2",
               "Rs3")

# unit_tests/models/unit_test_sorf.py:11-31
coordinates = np.array([[2.25571364, -0.38562082, 0.25521779],
                        [0.83507879, 1.9715759, -0.41464916],
                        [2.88876512, 0.84852166, 0.26907964],
                        [2.14876936, 2.01964345, -0.04776138],
                        [-3.48410053, 0.49229042, -0.10826158],
                        [0.92033708, -0.50883859, -0.10168934],
                        [0.21159328, 0.68818845, -0.42443103],
                        [-0.96446081, -1.83211358, -0.39899052],
                        [-1.65259035, 0.8639225, 1.35082265],
                        [0.88341369, -2.88346755, 0.19632983],
                        [0.22071292, -1.79338057, -0.09240105],
                        [-2.05297017, 0.69330798, 0.24948384],
                        [-1.12429142, 0.6204384, -0.81430244],
                        [0.29509341, -3.64658463, 0.43020677],
                        [2.66286461, -1.38969562, 0.4938589],
                        [0.26339145, 2.78767702, -0.91261049],
                        [3.94534538, 0.95482407, 0.58319346],
                        [2.74120081, 2.93792725, -0.25633347],
                        [-3.86742258, -0.54453643, -0.04496527],
                        [-4.02107013, 1.29272799, 0.46787286],
                        [-3.64746502, 0.93253809, -1.11074989]])
# unit_tests/models/unit_test_sorf.py:57
charges = np.array([6, 6, 6, 6, 6, 6, 6, 8, 8, 8, 6, 6, 8, 1, 1, 1, 1, 1, 1, 1, 1])
# unit_tests/models/unit_test_sorf.py:59-80 (the model's own printed fp32 outputs)
ref_energy = -406746.2188
ref_forces = np.array([[7.1108e+00, -2.3761e+01, 4.6022e+00],
                       [-3.9776e+01, -3.1590e+01, -2.3346e+01],
                       [5.2500e+00, 1.0356e+01, 1.2197e+01],
                       [5.0961e+01, 5.8797e+00, -1.4790e+01],
                       [-1.3412e+01, 4.5461e+01, -2.4878e+01],
                       [-8.1629e+00, 3.4137e+01, -1.9793e+00],
                       [-4.0663e+00, 2.8512e+00, 1.7828e+00],
                       [-1.2617e+01, -1.6348e+01, 6.7924e+00],
                       [1.1322e+01, 1.2017e+01, 5.5691e+01],
                       [4.8178e+01, -4.3340e+01, 2.7648e+01],
                       [-5.8656e+01, 2.4451e+01, -2.4338e+01],
                       [1.2962e+01, -2.4175e+01, -3.0994e+01],
                       [-1.1406e+01, 1.6746e+01, -7.4394e+00],
                       [2.1097e-01, 1.8720e+01, -1.2756e+01],
                       [1.5738e+01, 1.9531e+01, 1.7070e+00],
                       [1.0520e+01, -6.9458e+00, 1.7073e+01],
                       [-1.1871e+01, -3.0293e+00, -6.6352e+00],
                       [-1.0281e+01, -6.9400e+00, 1.3242e+01],
                       [5.4357e+00, 1.2351e+01, 4.4594e+00],
                       [2.7494e-02, -2.8147e+01, 8.2276e+00],
                       [2.5313e+00, -1.8224e+01, -6.2653e+00]])


def main():
    tree = model_files.read_attribute_tree(REF)
    out = {name: tree[name] for name in MODEL_TENSORS}
    out.update({name: tree["rep"][name] for name in REP_TENSORS})
    # +-1 diagonals travel as int8
    assert set(np.unique(out["Dmat"])) <= {-1.0, 1.0}
    out["Dmat"] = out["Dmat"].astype(np.int8)
    out["sigma"] = np.float64(tree["sigma"])
    out["npcas"] = np.int64(tree["npcas"])
    out["nstacks"] = np.int64(tree["nstacks"])
    out["coordinates"] = coordinates
    out["charges"] = charges
    out["ref_energy"] = np.float64(ref_energy)
    out["ref_forces"] = ref_forces
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
