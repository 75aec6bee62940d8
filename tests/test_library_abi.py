"""CPU-side checks of the C ABI: the built library loads, exports every symbol that
include/qmll.h declares with the argument count the ctypes table uses, and argument
validation refuses bad shapes before anything is launched (no GPU needed)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared():
    h = open(os.path.join(ROOT, "include", "qmll.h")).read()
    h = re.sub(r"/\*.*?\*/", "", h, flags=re.S)
    out = {}
    for m in re.finditer(r"^(?:int|size_t|double|const char\*)\s+(qmll_\w+)\s*\(([^;]*?)\)\s*;", h, re.M | re.S):
        args = m.group(2).strip()
        out[m.group(1)] = 0 if args in ("", "void") else len(args.split(","))
    return out


def test_header_and_ctypes_table_agree():
    from qml_lightning_amd import _lib
    decl = declared()
    assert len(decl) >= 20
    assert set(decl) == set(_lib.PROTOTYPES)
    for name, nargs in decl.items():
        assert nargs == len(_lib.PROTOTYPES[name]), name


def test_library_exports_every_declared_symbol():
    from qml_lightning_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.fail("libqmll.so has not been built: run python -c 'import __graft_entry__ as g; g.build()'")
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared():
        assert hasattr(handle, name), name
    assert _lib.lib().qmll_version() >= 1


def test_bad_arguments_are_refused_on_the_host():
    from qml_lightning_amd import _lib
    L = _lib.lib()
    null = ctypes.c_void_p(0)
    # non power of two -> the reference's message (hadamard_kernel.cu:730)
    rc = L.qmll_sorf_forward(ctypes.c_void_p(8), ctypes.c_void_p(8), 4, 12, 2, 1, 1.0, ctypes.c_void_p(8), null)
    assert rc == _lib.QMLL_ERR_NOT_POW2
    assert b"power of 2" in L.qmll_last_error()
    with pytest.raises(RuntimeError, match="power of 2"):
        _lib.check(rc)
    # null pointers with a non-empty shape
    assert L.qmll_sorf_forward(null, null, 4, 16, 2, 1, 1.0, null, null) == _lib.QMLL_ERR_INVALID
    assert L.qmll_gram_f64(null, null, 10, 16, null, null, null) == _lib.QMLL_ERR_INVALID
    assert L.qmll_gram_tile_f64(ctypes.c_void_p(8), null, 10, 16, 8, 4, ctypes.c_void_p(8), null, null) == _lib.QMLL_ERR_INVALID
    prm = _lib.FchlParams(0, 24, 20, 0.32, 2.7, 1.8, 13.4, 0.57, 6.0)
    args = [null] * 9 + [0, 5, 1, 12, null, null, ctypes.byref(prm), null, null]
    assert L.qmll_fchl19_forward(*args) == _lib.QMLL_ERR_INVALID
    # the all-elements force-feature entry: element count, projected dimension, null output
    elems = (_lib.DfElement * 9)()
    assert L.qmll_derivative_features_typed(elems, 9, 1.0, 3, 128, 4, 1, 2, 0, ctypes.c_void_p(8), null) == _lib.QMLL_ERR_INVALID
    assert b"at most 8" in L.qmll_last_error()
    assert L.qmll_derivative_features_typed(elems, 2, 1.0, 3, 512, 4, 1, 2, 0, ctypes.c_void_p(8), null) == _lib.QMLL_ERR_INVALID
    assert L.qmll_derivative_features_typed(elems, 2, 1.0, 3, 96, 4, 1, 2, 0, ctypes.c_void_p(8), null) == _lib.QMLL_ERR_NOT_POW2
    assert L.qmll_derivative_features_typed(elems, 2, 1.0, 3, 128, 4, 1, 2, 0, null, null) == _lib.QMLL_ERR_INVALID
    assert L.qmll_derivative_features_typed(elems, 2, 1.0, 3, 128, 4, 1, 2, 0, ctypes.c_void_p(8), null) == _lib.QMLL_ERR_INVALID  # null element pointers
    assert L.qmll_derivative_features_typed(elems, 2, 1.0, 3, 128, 4, 1, 0, 0, null, null) == _lib.QMLL_OK   # no molecules
    # the Cholesky entries
    assert L.qmll_cholesky_workspace_bytes(0) == 0 and L.qmll_cholesky_workspace_bytes(300) > 300 * 8
    assert L.qmll_cholesky_f64(null, 16, 16, null, null, null) == _lib.QMLL_ERR_INVALID
    assert L.qmll_cholesky_f64(ctypes.c_void_p(16), 16, 8, ctypes.c_void_p(16), ctypes.c_void_p(16), null) == _lib.QMLL_ERR_INVALID
    # the sort without a workspace refuses what its built-in counters cannot hold (ceil(A/256)*ne > 131072)
    assert L.qmll_sort_by_type_noalloc(ctypes.c_void_p(8), ctypes.c_void_p(8), 4097 * 256, 32, ctypes.c_void_p(8),
                                       ctypes.c_void_p(8), null) == _lib.QMLL_ERR_INVALID
    assert b"scratch" in L.qmll_last_error()
    # empty inputs are fine and launch nothing
    assert L.qmll_sorf_forward(null, null, 0, 16, 2, 1, 1.0, null, null) == _lib.QMLL_OK
    assert L.qmll_gram_f64(null, null, 0, 16, null, null, null) == _lib.QMLL_OK


def test_missing_library_fails_loudly(monkeypatch):
    from qml_lightning_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libqmll.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.lib()


def test_ops_are_registered_and_refuse_cpu_tensors():
    import torch
    import qml_lightning_amd  # noqa: F401
    assert hasattr(torch.ops.qml_lightning_fchl, "fchl_forwards")
    assert hasattr(torch.ops.qml_lightning_fchl, "get_fchl_and_derivative")
    assert hasattr(torch.ops.qml_lightning_sorf, "get_SORF_coefficients")
    assert hasattr(torch.ops.qml_lightning_sorf, "get_cos_features")
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        torch.ops.qml_lightning_sorf.get_SORF_coefficients(torch.zeros(2, 8), torch.ones(1, 2, 8), torch.tensor(1.0),
                                                           torch.tensor(1))


def test_cpp_operator_library_registers_every_operator():
    """libqmll_torch.so (TORCH_LIBRARY from C++, as the reference's torchscript_*.so) is what
    `import qml_lightning_amd` loads; the Python definitions are only its stand-in."""
    import torch
    import qml_lightning_amd  # noqa: F401
    from qml_lightning_amd import ops
    if os.environ.get("QML_LIGHTNING_AMD_PY_OPS") == "1" or "QML_LIGHTNING_AMD_LIB" in os.environ:
        pytest.skip("the Python operator definitions were asked for")
    assert os.path.exists(ops.TORCH_LIB_PATH), "libqmll_torch.so has not been built"
    assert ops.OPS_BACKEND == "c++"
    for name in ("fchl_forwards", "fchl_backwards", "get_fchl_and_derivative", "get_element_types",
                 "get_num_neighbours", "get_neighbour_list"):
        assert hasattr(torch.ops.qml_lightning_fchl, name), name
    for name in ("get_SORF_coefficients", "get_SORF_coefficients_backward", "get_cos_features",
                 "get_cos_features_backward", "sorf_energy", "sorf_energy_typed", "sort_by_type", "project_typed",
                 "project_typed_backward", "sorf_energy_sorted", "rff_energy_sorted", "fchl_sorf_energy",
                 "fchl_rff_energy"):
        assert hasattr(torch.ops.qml_lightning_sorf, name), name
    # schemas as TorchScript sees them: positional tensors, as in the reference
    schema = str(torch.ops.qml_lightning_fchl.fchl_forwards.default._schema)
    assert schema.count("Tensor") == 17      # 16 inputs, 1 output
    handle = ctypes.CDLL(ops.TORCH_LIB_PATH)
    assert handle.qmll_torch_ops_version() >= 1
