"""ctypes binding of libqmll.so, the C-ABI HIP library (declarations: include/qmll.h).

The library is the only compute path: if it is missing or a call fails this module
raises; there is no CPU or eager fallback.
"""
import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_double, c_float, c_int, c_longlong, c_size_t, c_void_p

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("QML_LIGHTNING_AMD_LIB", os.path.join(HERE, "libqmll.so"))

QMLL_OK = 0
QMLL_ERR_INVALID = -1
QMLL_ERR_LAUNCH = -2
QMLL_ERR_NOT_POW2 = -3


class FchlParams(Structure):
    """Mirror of struct qmll_fchl_params."""
    _fields_ = [("nspecies", c_int), ("nRs2", c_int), ("nRs3", c_int), ("eta2", c_float), ("eta3", c_float),
                ("two_body_decay", c_float), ("three_body_weight", c_float), ("three_body_decay", c_float),
                ("rcut", c_float)]


class DfElement(Structure):
    """Mirror of struct qmll_df_element (device pointers)."""
    _fields_ = [("cos_derivs", c_void_p), ("input_derivative", c_void_p), ("D", c_void_p), ("seg_offsets", c_void_p)]


P = c_void_p  # every device pointer and the stream travel as void*
_FCHL_COMMON = [P, P, P, P, P, P, P, P, P, c_int, c_int, c_int, c_int, P, P, POINTER(FchlParams)]

# name -> argtypes (restype is int unless listed in _RESTYPES)
PROTOTYPES = {
    "qmll_version": [],
    "qmll_last_error": [],
    "qmll_num_neighbours": [P, P, P, P, c_int, c_int, c_float, P, P],
    "qmll_neighbour_list": [P, P, P, P, c_int, c_int, c_int, c_float, P, P],
    "qmll_element_types": [P, P, P, c_int, c_int, c_int, P, P],
    "qmll_fchl19_forward": _FCHL_COMMON + [P, P],
    "qmll_fchl19_vjp": _FCHL_COMMON + [P, P, P],
    "qmll_fchl19_vjp_scaled": _FCHL_COMMON + [P, c_float, P, P],
    "qmll_fchl19_jacobian": _FCHL_COMMON + [P, P, P],
    "qmll_sorf_forward": [P, P, c_int, c_int, c_int, c_int, c_float, P, P],
    "qmll_sorf_adjoint": [P, P, c_int, c_int, c_int, c_int, c_float, P, P],
    "qmll_segment_offsets": [P, c_int, c_int, P, P],
    "qmll_cos_features_f32": [P, P, P, P, c_int, c_int, c_int, P, P],
    "qmll_cos_features_f64": [P, P, P, P, c_int, c_int, c_int, P, P],
    "qmll_cos_features_backward": [P, P, P, P, c_int, c_int, c_int, P, P],
    "qmll_sin_coeffs_f64": [P, P, c_int, c_int, P, P],
    "qmll_derivative_features": [P, c_double, P, P, P, P, c_int, c_int, c_int, c_int, c_int, c_int, P, P],
    "qmll_derivative_features_typed": [POINTER(DfElement), c_int, c_double, c_int, c_int, c_int, c_int, c_int, c_int, P, P],
    "qmll_sorf_energy_fused": [P, P, P, P, P, c_int, c_int, c_int, c_int, c_float, P, P, P],
    "qmll_sorf_energy_typed": [P, P, P, P, P, P, c_int, c_int, c_int, c_int, c_int, c_int, c_float, P, P, P],
    "qmll_sort_by_type_workspace": [c_int, c_int],
    "qmll_sort_by_type": [P, P, c_int, c_int, P, c_size_t, P, P, P],
    "qmll_sort_atoms_workspace": [c_int, c_int],
    "qmll_sort_atoms_by_type": [P, P, P, c_int, c_int, c_int, P, c_size_t, P, P, P],
    "qmll_sort_by_type_noalloc": [P, P, c_int, c_int, P, P, P],
    "qmll_reductor_presplit_bytes": [c_int, c_int, c_int],
    "qmll_reductor_presplit": [P, c_int, c_int, c_int, P, c_size_t, P],
    "qmll_project_typed": [P, P, P, P, P, c_int, c_int, c_int, c_int, P, P],
    "qmll_project_typed_rows": [P, P, P, P, c_int, c_int, c_int, c_int, c_int, P, P],
    "qmll_project_typed_backward": [P, P, P, P, P, P, c_int, c_int, c_int, c_int, c_int, P, P],
    "qmll_project_typed_backward_sums": [P, P, P, P, P, P, c_int, c_int, c_int, c_int, c_int, P, P, c_int, c_int, P, P],
    "qmll_prepare_batch": [P, P, P, c_int, P, c_int, P, P, c_int, c_int, c_int, P, c_size_t, P, P, P, P, P, c_size_t, P],
    "qmll_sorf_energy_sorted": [P, P, P, P, P, P, P, c_int, c_int, c_int, c_int, c_int, c_float, P, P, P],
    "qmll_rff_features": [P, P, P, P, c_int, c_int, c_int, c_int, P, P],
    "qmll_rff_derivative_features": [P, P, P, P, P, P, c_int, c_int, c_int, c_int, c_int, P, P],
    "qmll_rff_presplit_bytes": [c_int, c_int, c_int],
    "qmll_rff_presplit": [P, c_int, c_int, c_int, P, c_size_t, P],
    "qmll_rff_energy_sorted": [P, P, P, P, P, P, c_int, c_int, c_int, c_int, P, P, P],
    "qmll_gram_f64": [P, P, c_int, c_int, P, P, P],
    "qmll_gram_upper_f64": [P, P, c_int, c_int, P, P, P],
    "qmll_gram_workspace_bytes": [],
    "qmll_gram_upper_ws_f64": [P, P, c_int, c_int, P, P, P, c_size_t, P],
    "qmll_gram_mirror_f64": [P, c_int, P],
    "qmll_cholesky_workspace_bytes": [c_int],
    "qmll_cholesky_f64": [P, c_int, c_longlong, P, P, P],
    "qmll_cholesky_solve_f64": [P, c_int, c_longlong, P, P, P],
    "qmll_gram_tile_f64": [P, P, c_int, c_int, c_int, c_int, P, P, P],
    "qmll_matmul_and_reduce": [P, P, c_int, c_int, c_int, P, P],
    "qmll_probe_fill": [P, c_size_t, c_float, P],
    "qmll_probe_copy": [P, P, c_size_t, P],
    "qmll_probe_out_bytes": [],
    "qmll_probe_rate": [c_int, c_int, c_int, P, P],
    "qmll_probe_mix": [c_int, c_int, c_int, P, P],
}
_RESTYPES = {"qmll_last_error": c_char_p, "qmll_rff_presplit_bytes": c_size_t, "qmll_reductor_presplit_bytes": c_size_t, "qmll_sort_by_type_workspace": c_size_t, "qmll_sort_atoms_workspace": c_size_t,
             "qmll_cholesky_workspace_bytes": c_size_t, "qmll_gram_workspace_bytes": c_size_t,
             "qmll_probe_out_bytes": c_size_t, "qmll_probe_rate": c_double,
             "qmll_probe_mix": c_double}

_lib = None


def lib():
    """The loaded library (loaded once).  Raises RuntimeError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "qml_lightning_amd: %s not found -- build it with `python -m qml_lightning_amd.build` "
                "(there is no fallback path)" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        for name, argtypes in PROTOTYPES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = _RESTYPES.get(name, c_int)
        _lib = handle
    return _lib


def check(rc, what=""):
    """Turn a negative status into the exception the reference raises for the same fault:
    RuntimeError carrying the library's message (TORCH_CHECK -> RuntimeError there)."""
    if rc != QMLL_OK:
        msg = lib().qmll_last_error().decode("utf-8", "replace")
        raise RuntimeError(msg or ("%s failed with status %d" % (what, rc)))
