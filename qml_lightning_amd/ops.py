"""Tensor-level entry points over libqmll and the `torch.ops` the reference registers.

Two layers:
  * plain functions (`fchl_forward`, `sorf_forward`, ...): allocate outputs with torch,
    pass `data_ptr()`s and the current HIP stream to the C ABI, return tensors;
  * `torch.library` definitions of the operators the reference's TorchScript libraries
    export (qml_lightning/cuda/torchscript/FCHL19.cpp:318-333, SORF.cpp:138-150), with
    autograd, so that `torch.ops.qml_lightning_fchl.fchl_forwards` etc. resolve from Python
    and from TorchScript exactly as they do with the reference's `.so` files loaded.

Everything here requires the tensors to live on a HIP device ("cuda" in PyTorch-ROCm);
there is no CPU implementation.
"""
import ctypes
import math
import os
import weakref

import torch

from . import _lib
from ._lib import FchlParams, check

_P = ctypes.c_void_p


def _ptr(t):
    """Device address of a tensor for the C ABI (NULL for None).  A host tensor is refused
    here, whatever the caller checked: its address handed to a kernel is a GPU memory fault."""
    if t is None:
        return _P(0)
    if not t.is_cuda:
        raise RuntimeError("expected a CUDA tensor, got one on %s" % t.device)
    return _P(t.data_ptr())


_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_RAW_DEVICE = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """Handle of torch's current stream on the current device.  The raw accessors cost well under a
    microsecond; torch.cuda.current_stream() builds a Stream object and re-checks device
    availability on every call (8 us), seven times per predict step."""
    if _RAW_STREAM is not None and _RAW_DEVICE is not None:
        return _P(_RAW_STREAM(_RAW_DEVICE()))
    return _P(torch.cuda.current_stream().cuda_stream)


def _need_cuda(t, name):
    # same fault, same exception type as the reference's TORCH_CHECK (fchl_cuda.cpp:30-34)
    if not t.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor" % name)


def _f32(t):
    return t.contiguous() if t.dtype == torch.float32 else t.float().contiguous()


def _i32(t):
    return t.contiguous() if t.dtype == torch.int32 else t.to(torch.int32).contiguous()


def _cells(cell, inv_cell):
    """[B,3,3] pair or None; an empty [0,3,3] tensor means 'no periodic images'
    (reference: fchl_cuda_kernel.cu:548)."""
    if cell is None or cell.numel() == 0:
        return None, None
    return _f32(cell), _f32(inv_cell)


def _batched(X, Z=None):
    if X.dim() == 2:                       # fchl_cuda.cpp:72-76
        X = X.unsqueeze(0)
    if Z is not None and Z.dim() == 1:
        Z = Z.unsqueeze(0)
    return X, Z


def _scalar(v):
    return float(v.item()) if torch.is_tensor(v) else float(v)


def make_params(nspecies, Rs2, Rs3, eta2, eta3, two_body_decay, three_body_weight, three_body_decay, rcut):
    return FchlParams(int(nspecies), int(Rs2.shape[0]), int(Rs3.shape[0]), _scalar(eta2), _scalar(eta3),
                      _scalar(two_body_decay), _scalar(three_body_weight), _scalar(three_body_decay), _scalar(rcut))


# ---------------------------------------------------------------------------------------
# neighbours / element types
# ---------------------------------------------------------------------------------------
def num_neighbours(X, natoms, rcut, cell=None, inv_cell=None):
    _need_cuda(X, "coordinates")
    X, _ = _batched(X)
    X = _f32(X)
    natoms = _i32(natoms)
    cell, inv_cell = _cells(cell, inv_cell)
    B, n, _ = X.shape
    out = torch.empty((B, n), dtype=torch.int32, device=X.device)
    check(_lib.lib().qmll_num_neighbours(_ptr(X), _ptr(natoms), _ptr(cell), _ptr(inv_cell), B, n, _scalar(rcut),
                                         _ptr(out), _stream()), "qmll_num_neighbours")
    return out


def neighbour_list(X, natoms, max_neighbours, rcut, cell=None, inv_cell=None):
    _need_cuda(X, "coordinates")
    X, _ = _batched(X)
    X = _f32(X)
    natoms = _i32(natoms)
    cell, inv_cell = _cells(cell, inv_cell)
    B, n, _ = X.shape
    nn = int(max_neighbours.item()) if torch.is_tensor(max_neighbours) else int(max_neighbours)
    out = torch.empty((B, n, nn), dtype=torch.int32, device=X.device)
    check(_lib.lib().qmll_neighbour_list(_ptr(X), _ptr(natoms), _ptr(cell), _ptr(inv_cell), B, n, nn, _scalar(rcut),
                                         _ptr(out), _stream()), "qmll_neighbour_list")
    return out


def element_types(X, Z, natoms, species):
    _need_cuda(X, "coordinates")
    _need_cuda(Z, "charges")
    _need_cuda(species, "species")
    X, Z = _batched(X, Z)
    Z = _f32(Z)
    natoms = _i32(natoms)
    species = _f32(species)
    B, n = Z.shape
    out = torch.empty((B, n), dtype=torch.int32, device=Z.device)
    check(_lib.lib().qmll_element_types(_ptr(Z), _ptr(natoms), _ptr(species), B, n, species.shape[0], _ptr(out),
                                        _stream()), "qmll_element_types")
    return out


# ---------------------------------------------------------------------------------------
# FCHL19
# ---------------------------------------------------------------------------------------
def _fchl_args(X, types, cell, inv_cell, atomIDs, molIDs, natoms, nlist, nneigh, Rs2, Rs3, prm):
    B, n, _ = X.shape
    nn_stride = int(nlist.shape[2]) if nlist is not None else 0
    return [_ptr(X), _ptr(types), _ptr(cell), _ptr(inv_cell), _ptr(atomIDs), _ptr(molIDs), _ptr(natoms),
            _ptr(nlist), _ptr(nneigh), nn_stride, int(atomIDs.shape[0]), B, n, _ptr(Rs2), _ptr(Rs3),
            ctypes.byref(prm)]


def _fchl_prepare(X, types, cell, inv_cell, atomIDs, molIDs, natoms, nlist, nneigh, Rs2, Rs3):
    _need_cuda(X, "coordinates")
    X, _ = _batched(X)
    X = _f32(X)
    if types.dim() == 1:
        types = types.unsqueeze(0)
    types = _i32(types)
    cell, inv_cell = _cells(cell, inv_cell)
    atomIDs, molIDs, natoms = _i32(atomIDs), _i32(molIDs), _i32(natoms)
    if nlist is not None:
        nlist, nneigh = _i32(nlist), _i32(nneigh)
        if nlist.shape[2] == 0:
            nlist, nneigh = None, None
    return X, types, cell, inv_cell, atomIDs, molIDs, natoms, nlist, nneigh, _f32(Rs2), _f32(Rs3)


def repsize(prm):
    return prm.nspecies * prm.nRs2 + prm.nspecies * (prm.nspecies + 1) * prm.nRs3


def fchl_forward(X, types, cell, inv_cell, atomIDs, molIDs, natoms, Rs2, Rs3, prm, nlist=None, nneigh=None,
                 zero_fill=True):
    """rep f32 [B,n,R]; zero rows for padded slots (fchl_cuda.cpp:83).  zero_fill=False leaves the rows
    of slots that are not listed unwritten (the kernel writes every bin of a listed atom's row): for
    callers that read listed rows only."""
    X, types, cell, inv_cell, atomIDs, molIDs, natoms, nlist, nneigh, Rs2, Rs3 = _fchl_prepare(
        X, types, cell, inv_cell, atomIDs, molIDs, natoms, nlist, nneigh, Rs2, Rs3)
    B, n, _ = X.shape
    rep = (torch.zeros if zero_fill else torch.empty)((B, n, repsize(prm)), dtype=torch.float32, device=X.device)
    args = _fchl_args(X, types, cell, inv_cell, atomIDs, molIDs, natoms, nlist, nneigh, Rs2, Rs3, prm)
    check(_lib.lib().qmll_fchl19_forward(*args, _ptr(rep), _stream()), "qmll_fchl19_forward")
    return rep


def fchl_vjp(grad_rep, X, types, cell, inv_cell, atomIDs, molIDs, natoms, Rs2, Rs3, prm, nlist=None, nneigh=None,
             out=None, scale=1.0):
    """grad_X f32 [B,n,3] (fchl_cuda.cpp:196), times `scale` (-1: forces from an energy gradient).
    out: a zero-filled contiguous f32 [B,n,3] to add into."""
    X, types, cell, inv_cell, atomIDs, molIDs, natoms, nlist, nneigh, Rs2, Rs3 = _fchl_prepare(
        X, types, cell, inv_cell, atomIDs, molIDs, natoms, nlist, nneigh, Rs2, Rs3)
    B, n, _ = X.shape
    grad_rep = _f32(grad_rep).reshape(B, n, repsize(prm))
    if out is None:
        gX = torch.zeros((B, n, 3), dtype=torch.float32, device=X.device)
    else:
        gX = out
        if gX.dtype != torch.float32 or tuple(gX.shape) != (B, n, 3) or not gX.is_contiguous():
            raise RuntimeError("fchl_vjp: out must be a contiguous float32 [%d, %d, 3] tensor" % (B, n))
    args = _fchl_args(X, types, cell, inv_cell, atomIDs, molIDs, natoms, nlist, nneigh, Rs2, Rs3, prm)
    check(_lib.lib().qmll_fchl19_vjp_scaled(*args, _ptr(grad_rep), float(scale), _ptr(gX), _stream()), "qmll_fchl19_vjp")
    return gX


def fchl_jacobian(X, types, cell, inv_cell, atomIDs, molIDs, natoms, Rs2, Rs3, prm, nlist=None, nneigh=None,
                  with_rep=True):
    """(rep f32 [B,n,R] or None, jac f32 [B,n,n,3,R]) (fchl_cuda.cpp:186-187)."""
    X, types, cell, inv_cell, atomIDs, molIDs, natoms, nlist, nneigh, Rs2, Rs3 = _fchl_prepare(
        X, types, cell, inv_cell, atomIDs, molIDs, natoms, nlist, nneigh, Rs2, Rs3)
    B, n, _ = X.shape
    R = repsize(prm)
    rep = torch.zeros((B, n, R), dtype=torch.float32, device=X.device) if with_rep else None
    jac = torch.zeros((B, n, n, 3, R), dtype=torch.float32, device=X.device)
    args = _fchl_args(X, types, cell, inv_cell, atomIDs, molIDs, natoms, nlist, nneigh, Rs2, Rs3, prm)
    check(_lib.lib().qmll_fchl19_jacobian(*args, _ptr(rep), _ptr(jac), _stream()), "qmll_fchl19_jacobian")
    return rep, jac


# ---------------------------------------------------------------------------------------
# SORF / features
# ---------------------------------------------------------------------------------------
def sorf_forward(u, D, normalisation, ntransforms):
    """[A,d] x [T,S,d] -> [A,S,d] (hadamard_cuda.cpp:47-56)."""
    _need_cuda(u, "input")
    _need_cuda(D, "dmatrix")
    u, D = _f32(u), _f32(D)
    A, d = u.shape
    T, S = int(ntransforms), int(D.shape[1])
    if T > D.shape[0]:
        raise RuntimeError("ntransforms (%d) exceeds the %d diagonals given" % (T, D.shape[0]))
    if D.dim() != 3 or D.shape[2] != d:
        raise RuntimeError("sorf_forward: input is %s, diagonals are %s: the last dimensions must agree"
                           % (tuple(u.shape), tuple(D.shape)))
    out = torch.empty((A, S, d), dtype=torch.float32, device=u.device)
    check(_lib.lib().qmll_sorf_forward(_ptr(u), _ptr(D), A, d, S, T, float(normalisation), _ptr(out), _stream()),
          "qmll_sorf_forward")
    return out


def sorf_adjoint(g, D, normalisation, ntransforms):
    """[A,S,d] -> [A,d] (hadamard_cuda.cpp:58-70)."""
    _need_cuda(g, "input")
    _need_cuda(D, "dmatrix")
    g, D = _f32(g), _f32(D)
    A, S, d = g.shape
    T = int(ntransforms)
    if D.dim() != 3 or T > D.shape[0] or D.shape[1] != S or D.shape[2] != d:
        raise RuntimeError("sorf_adjoint: gradient is %s, diagonals are %s, %d transforms" % (tuple(g.shape), tuple(D.shape), T))
    out = torch.empty((A, d), dtype=torch.float32, device=g.device)
    check(_lib.lib().qmll_sorf_adjoint(_ptr(g), _ptr(D), A, d, S, T, float(normalisation), _ptr(out), _stream()),
          "qmll_sorf_adjoint")
    return out


def segment_offsets(mol_index, nmol):
    """int32 [nmol+2]: first atom of each molecule of an ascending molecule index, then a
    flag that is non-zero when the index is not ascending (checked on the device)."""
    mol_index = _i32(mol_index)
    seg = torch.zeros(int(nmol) + 2, dtype=torch.int32, device=mol_index.device)
    check(_lib.lib().qmll_segment_offsets(_ptr(mol_index), int(mol_index.shape[0]), int(nmol), _ptr(seg), _stream()),
          "qmll_segment_offsets")
    return seg


def cos_features(coeffs, bias, nmol, mol_index, out=None):
    """f32 [nmol,F] (new, zero-initialised) or accumulate into a given f32/f64 tensor."""
    _need_cuda(coeffs, "coeffs")
    _need_cuda(bias, "b")
    _need_cuda(mol_index, "batch_indexes")
    coeffs, bias, mol_index = _f32(coeffs), _f32(bias), _i32(mol_index)
    A, F = coeffs.shape
    if bias.numel() != F or mol_index.numel() != A:
        raise RuntimeError("cos_features: coefficients are %s, bias has %d entries, batch_indexes %d"
                           % (tuple(coeffs.shape), bias.numel(), mol_index.numel()))
    if out is None:
        out = torch.zeros((int(nmol), F), dtype=torch.float32, device=coeffs.device)
    if not out.is_contiguous() or out.dim() != 2 or out.shape[1] != F:
        raise RuntimeError("feature matrix must be contiguous with %d columns" % F)
    fn = _lib.lib().qmll_cos_features_f64 if out.dtype == torch.float64 else _lib.lib().qmll_cos_features_f32
    seg = segment_offsets(mol_index, out.shape[0]) if A > 0 else None
    check(fn(_ptr(coeffs), _ptr(bias), _ptr(mol_index), _ptr(seg), A, F, int(out.shape[0]), _ptr(out), _stream()),
          "qmll_cos_features")
    return out


def cos_features_backward(gZ, coeffs, bias, nmol, mol_index):
    gZ, coeffs, bias, mol_index = _f32(gZ), _f32(coeffs), _f32(bias), _i32(mol_index)
    A, F = coeffs.shape
    if bias.numel() != F or mol_index.numel() != A or gZ.dim() != 2 or gZ.shape[1] != F:
        raise RuntimeError("cos_features_backward: coefficients are %s, gradient %s, bias has %d entries, batch_indexes %d"
                           % (tuple(coeffs.shape), tuple(gZ.shape), bias.numel(), mol_index.numel()))
    out = torch.empty((A, F), dtype=torch.float32, device=coeffs.device)
    check(_lib.lib().qmll_cos_features_backward(_ptr(gZ), _ptr(coeffs), _ptr(bias), _ptr(mol_index), A, F,
                                                int(gZ.shape[0]), _ptr(out), _stream()), "qmll_cos_features_backward")
    return out


def sin_coeffs(coeffs, bias, out):
    coeffs, bias = _f32(coeffs), _f32(bias)
    A, F = coeffs.shape
    if bias.numel() != F:
        raise RuntimeError("sin_coeffs: bias has %d entries for %d features" % (bias.numel(), F))
    if out.dtype != torch.float64 or not out.is_contiguous() or tuple(out.shape) != (A, F):
        raise RuntimeError("sin_coeffs output must be a contiguous float64 [A,F] tensor")
    check(_lib.lib().qmll_sin_coeffs_f64(_ptr(coeffs), _ptr(bias), A, F, _ptr(out), _stream()), "qmll_sin_coeffs_f64")
    return out


def derivative_features(cos_derivs, normalisation, D, input_derivatives, mol_index, G, molecule_major=False):
    """G += force-feature rows of one element.  molecule_major=True promises that
    mol_index is non-decreasing (atoms grouped by molecule): the atomic-free kernel is
    used, with segment offsets found on the device."""
    D, u, mol_index = _f32(D), _f32(input_derivatives), _i32(mol_index)
    A, n, _, d = u.shape
    T, S, _ = D.shape
    if (cos_derivs.dtype != torch.float64 or not cos_derivs.is_contiguous() or G.dtype != torch.float64
            or not G.is_contiguous()):
        raise RuntimeError("derivative features need contiguous float64 cos_derivs and output")
    if G.shape[1] != n or G.shape[3] != S * d:
        raise RuntimeError("feature_derivatives has shape %s, expected [nmol,%d,3,%d]" % (tuple(G.shape), n, S * d))
    nmol = int(G.shape[0])
    seg = None
    if molecule_major:
        bounds = torch.arange(nmol + 1, dtype=torch.int32, device=u.device)
        seg = torch.searchsorted(mol_index, bounds).to(torch.int32)
    check(_lib.lib().qmll_derivative_features(_ptr(cos_derivs), float(normalisation), _ptr(mol_index), _ptr(seg),
                                              _ptr(u), _ptr(D), A, n, d, S, T, nmol, _ptr(G), _stream()),
          "qmll_derivative_features")
    return G


def derivative_features_typed(items, normalisation, G, overwrite=False):
    """G += force-feature rows of every element of the batch in one launch.  items: one tuple
    (cos_derivs f64 [A_e,F], D f32 [T,S,d], input_derivatives f32 [A_e,n,3,d], mol_index i32 [A_e],
    non-decreasing) per element.  Each G element is read and written once, instead of once per
    element and atom chunk as with `derivative_features`; with overwrite, G = those rows and is
    only written (it may come from torch.empty).  64 <= d <= 256, at most 8 elements."""
    if not items:
        return G.zero_() if overwrite else G
    if G.dtype != torch.float64 or not G.is_contiguous():
        raise RuntimeError("derivative features need a contiguous float64 output")
    nmol, n = int(G.shape[0]), int(G.shape[1])
    keep, structs = [], (_lib.DfElement * len(items))()
    T = S = d = None
    bounds = torch.arange(nmol + 1, dtype=torch.int32, device=G.device)
    for k, (cos_derivs, D, u, mol_index) in enumerate(items):
        D, u, mol_index = _f32(D), _f32(u), _i32(mol_index)
        if cos_derivs.dtype != torch.float64 or not cos_derivs.is_contiguous():
            raise RuntimeError("derivative features need contiguous float64 cos_derivs")
        if T is None:
            T, S, d = (int(v) for v in D.shape)
        if tuple(D.shape) != (T, S, d) or tuple(u.shape[1:]) != (n, 3, d) or cos_derivs.shape != (u.shape[0], S * d):
            raise RuntimeError("derivative_features_typed: element %d does not fit [T,S,d] = %s, n = %d" % (k, (T, S, d), n))
        seg = torch.searchsorted(mol_index, bounds).to(torch.int32)
        keep.append((cos_derivs, D, u, seg))
        structs[k].cos_derivs = cos_derivs.data_ptr()
        structs[k].input_derivative = u.data_ptr()
        structs[k].D = D.data_ptr()
        structs[k].seg_offsets = seg.data_ptr()
    if G.shape[3] != S * d:
        raise RuntimeError("feature_derivatives has shape %s, expected [nmol,%d,3,%d]" % (tuple(G.shape), n, S * d))
    check(_lib.lib().qmll_derivative_features_typed(structs, len(items), float(normalisation), n, d, S, T, nmol,
                                                    int(bool(overwrite)), _ptr(G), _stream()),
          "qmll_derivative_features_typed")
    return G


def sorf_energy_fused(x, D, bias, alpha, out_index, normalisation, ntransforms, e_atom, with_grad=True):
    """Per-atom energies written into e_atom[out_index]; returns d e_atom / d x or None."""
    x, D, bias, alpha = _f32(x), _f32(D), _f32(bias), _f32(alpha)
    A, d = x.shape
    S, T = int(D.shape[1]), int(ntransforms)
    if D.dim() != 3 or D.shape[2] != d or T > D.shape[0] or bias.numel() != S * d or alpha.numel() != S * d:
        raise RuntimeError("sorf_energy_fused: x %s, diagonals %s, bias with %d and alpha with %d entries do not fit together"
                           % (tuple(x.shape), tuple(D.shape), bias.numel(), alpha.numel()))
    gx = torch.empty((A, d), dtype=torch.float32, device=x.device) if with_grad else None
    check(_lib.lib().qmll_sorf_energy_fused(_ptr(x), _ptr(D), _ptr(bias), _ptr(alpha), _ptr(out_index), A, d, S, T,
                                            float(normalisation), _ptr(e_atom), _ptr(gx), _stream()),
          "qmll_sorf_energy_fused")
    return gx


def sorf_energy_typed(x_all, types, atom_slots, Dmat, bias, alpha, normalisation, ntransforms, with_grad=True):
    """All elements in one launch.  x_all [N, ne*d], types int32 [N], atom_slots int32 [A],
    Dmat [ne,T,S,d], bias [ne,F], alpha [F] -> (e_slots [N], gx_all [N, ne*d] or None)."""
    x_all, Dmat, bias, alpha = _f32(x_all), _f32(Dmat), _f32(bias), _f32(alpha)
    types, atom_slots = _i32(types).reshape(-1), _i32(atom_slots)
    ne, Tn, S, d = Dmat.shape
    N = x_all.shape[0]
    if x_all.shape[1] != ne * d or types.shape[0] != N:
        raise RuntimeError("sorf_energy_typed: x_all is %s, expected [%d, %d]" % (tuple(x_all.shape), types.shape[0], ne * d))
    T = int(ntransforms)
    if T != Tn:
        raise RuntimeError("sorf_energy_typed: %d diagonals stored per stack, %d transforms asked for" % (Tn, T))
    if tuple(bias.shape) != (ne, S * d) or alpha.numel() != S * d:
        raise RuntimeError("sorf_energy_typed: bias %s / alpha with %d entries do not fit %d elements and %d features"
                           % (tuple(bias.shape), alpha.numel(), ne, S * d))
    e_slots = torch.zeros(N, dtype=torch.float32, device=x_all.device)
    gx = torch.zeros((N, ne * d), dtype=torch.float32, device=x_all.device) if with_grad else None
    check(_lib.lib().qmll_sorf_energy_typed(_ptr(x_all), _ptr(types), _ptr(atom_slots), _ptr(Dmat), _ptr(bias),
                                            _ptr(alpha), int(atom_slots.shape[0]), N, ne, d, S, T, float(normalisation),
                                            _ptr(e_slots), _ptr(gx), _stream()), "qmll_sorf_energy_typed")
    return e_slots, gx


# ---------------------------------------------------------------------------------------
# element-sorted projection + fused energy
# ---------------------------------------------------------------------------------------
def sort_by_type(types, slots, ne):
    """Stable sort of the real atoms' slots by element type -> (sorted_slots [A], type_offsets [ne+1])."""
    types, slots = _i32(types).reshape(-1), _i32(slots).reshape(-1)
    A = int(slots.shape[0])
    sorted_slots = torch.empty(A, dtype=torch.int32, device=types.device)
    offsets = torch.empty(ne + 1, dtype=torch.int32, device=types.device)
    nbytes = int(_lib.lib().qmll_sort_by_type_workspace(A, ne))
    work = torch.empty(max(nbytes // 4, 1), dtype=torch.int32, device=types.device)
    check(_lib.lib().qmll_sort_by_type(_ptr(types), _ptr(slots), A, int(ne), _ptr(work), nbytes, _ptr(sorted_slots),
                                       _ptr(offsets), _stream()), "qmll_sort_by_type")
    return sorted_slots, offsets


def sort_atoms_by_type(types, atomIDs, molIDs, n, ne):
    """`sort_by_type` of the listed atoms of a padded [B, n] batch, slot = molIDs * n + atomIDs; one
    launch and no workspace up to 1024 atoms."""
    types, atomIDs, molIDs = _i32(types).reshape(-1), _i32(atomIDs).reshape(-1), _i32(molIDs).reshape(-1)
    A = int(atomIDs.shape[0])
    if int(molIDs.shape[0]) != A:
        raise RuntimeError("sort_atoms_by_type: %d atom indices, %d molecule indices" % (A, int(molIDs.shape[0])))
    sorted_slots = torch.empty(A, dtype=torch.int32, device=types.device)
    offsets = torch.empty(ne + 1, dtype=torch.int32, device=types.device)
    nbytes = int(_lib.lib().qmll_sort_atoms_workspace(A, ne))
    work = torch.empty(nbytes // 4, dtype=torch.int32, device=types.device) if nbytes else None
    check(_lib.lib().qmll_sort_atoms_by_type(_ptr(types), _ptr(atomIDs), _ptr(molIDs), int(n), A, int(ne), _ptr(work), nbytes,
                                             _ptr(sorted_slots), _ptr(offsets), _stream()), "qmll_sort_atoms_by_type")
    return sorted_slots, offsets


def prepare_batch(Z, natoms, species, atomIDs, molIDs, model_species=None, zero_count=0):
    """What the fused predict chain needs before its first compute kernel, in one launch for small
    batches: (types [B,n] by `species`, sort_types [B,n] by `model_species` (types itself when that is
    None), sorted_slots [A], type_offsets [ne+1], zeroed f32 [zero_count])."""
    _need_cuda(Z, "charges")
    Zb = _f32(Z if Z.dim() == 2 else Z.unsqueeze(0))
    natoms, species = _i32(natoms), _f32(species)
    atomIDs, molIDs = _i32(atomIDs).reshape(-1), _i32(molIDs).reshape(-1)
    B, n = Zb.shape
    A = int(atomIDs.shape[0])
    own = model_species is not None and model_species.numel() > 0
    msp = _f32(model_species) if own else None
    ne = int(msp.shape[0]) if own else int(species.shape[0])
    dev = Zb.device
    types = torch.empty((B, n), dtype=torch.int32, device=dev)
    sort_types = torch.empty((B, n), dtype=torch.int32, device=dev) if own else types
    sorted_slots = torch.empty(A, dtype=torch.int32, device=dev)
    offsets = torch.empty(ne + 1, dtype=torch.int32, device=dev)
    zero = torch.empty(int(zero_count), dtype=torch.float32, device=dev)
    nbytes = int(_lib.lib().qmll_sort_atoms_workspace(A, ne))
    work = torch.empty(nbytes // 4, dtype=torch.int32, device=dev) if nbytes else None
    check(_lib.lib().qmll_prepare_batch(_ptr(Zb), _ptr(natoms), _ptr(species), int(species.shape[0]), _ptr(msp), ne,
                                        _ptr(atomIDs), _ptr(molIDs), B, n, A, _ptr(work), nbytes, _ptr(types),
                                        _ptr(sort_types) if own else None, _ptr(sorted_slots), _ptr(offsets), _ptr(zero),
                                        int(zero_count), _stream()), "qmll_prepare_batch")
    return types, sort_types, sorted_slots, offsets, zero


def reductor_presplit(reductors):
    """The reductors [ne,R,d] in the form the fp16 matrix-core projection kernels multiply with
    (qmll_reductor_presplit): an opaque uint8 device buffer, or None when no kernel takes one."""
    reductors = _f32(reductors)
    ne, R, d = reductors.shape
    nbytes = int(_lib.lib().qmll_reductor_presplit_bytes(ne, R, d))
    if nbytes == 0:
        return None
    out = torch.empty(nbytes, dtype=torch.uint8, device=reductors.device)
    check(_lib.lib().qmll_reductor_presplit(_ptr(reductors), ne, R, d, _ptr(out), nbytes, _stream()),
          "qmll_reductor_presplit")
    return out


#: from this many atoms on the projections are handed the prepared reductors (below, the
#: one-workgroup-per-atom kernels run, which read the fp32 reductors)
SPLIT_FROM_ATOMS = 2049


def _split_for(reductors, A):
    return presplit_cached(reductors, "reductor", reductor_presplit) if A >= SPLIT_FROM_ATOMS else None


def project_typed(rep, sorted_slots, type_offsets, reductors):
    """x [A,d]: row a = rep[sorted_slots[a]] . reductors[type of a] (rep [N,R], reductors [ne,R,d])."""
    rep, reductors = _f32(rep), _f32(reductors)
    sorted_slots, type_offsets = _i32(sorted_slots), _i32(type_offsets)
    ne, R, d = reductors.shape
    if rep.dim() != 2 or rep.shape[1] != R or type_offsets.shape[0] != ne + 1:
        raise RuntimeError("project_typed: rep %s, reductors %s, %d offsets do not fit together"
                           % (tuple(rep.shape), tuple(reductors.shape), type_offsets.shape[0]))
    A = int(sorted_slots.shape[0])
    x = torch.empty((A, d), dtype=torch.float32, device=rep.device)
    check(_lib.lib().qmll_project_typed(_ptr(rep), _ptr(sorted_slots), _ptr(type_offsets), _ptr(reductors),
                                        _ptr(_split_for(reductors, A)), A, ne, R, d, _ptr(x), _stream()),
          "qmll_project_typed")
    return x


def project_typed_rows(rows, sorted_slots, type_offsets, reductors, group):
    """x [A*group,d]: x[a*group+g] = rows[sorted_slots[a]*group+g] . reductors[type of a]
    (rows [N*group,R], `group` consecutive rows per slot; reductors [ne,R,d])."""
    rows, reductors = _f32(rows), _f32(reductors)
    sorted_slots, type_offsets = _i32(sorted_slots), _i32(type_offsets)
    ne, R, d = reductors.shape
    group = int(group)
    if rows.dim() != 2 or rows.shape[1] != R or type_offsets.shape[0] != ne + 1 or group < 1 or rows.shape[0] % group:
        raise RuntimeError("project_typed_rows: rows %s, reductors %s, %d offsets, group %d do not fit together"
                           % (tuple(rows.shape), tuple(reductors.shape), type_offsets.shape[0], group))
    A = int(sorted_slots.shape[0])
    x = torch.empty((A * group, d), dtype=torch.float32, device=rows.device)
    check(_lib.lib().qmll_project_typed_rows(_ptr(rows), _ptr(sorted_slots), _ptr(type_offsets), _ptr(reductors), A, ne, R,
                                             d, group, _ptr(x), _stream()), "qmll_project_typed_rows")
    return x


def project_typed_backward(gx, sorted_slots, type_offsets, reductors, types, nslots):
    """g_rep [nslots,R] with g_rep[sorted_slots[a]] = gx[a] . reductors[type]^T, zero elsewhere."""
    gx, reductors = _f32(gx), _f32(reductors)
    sorted_slots, type_offsets, types = _i32(sorted_slots), _i32(type_offsets), _i32(types).reshape(-1)
    ne, R, d = reductors.shape
    A, N = int(sorted_slots.shape[0]), int(nslots)
    if gx.shape[0] != A or gx.shape[1] != d or types.shape[0] != N:
        raise RuntimeError("project_typed_backward: gx %s for %d atoms, d=%d" % (tuple(gx.shape), A, d))
    if A == N:
        # every slot holds a real atom: the kernel writes every row of a known element and
        # zeroes the rows of unknown ones
        g_rep = torch.empty((N, R), dtype=torch.float32, device=gx.device)
        tz = types
    else:
        g_rep = torch.zeros((N, R), dtype=torch.float32, device=gx.device)
        tz = None
    check(_lib.lib().qmll_project_typed_backward(_ptr(gx), _ptr(sorted_slots), _ptr(type_offsets), _ptr(reductors),
                                                 _ptr(_split_for(reductors, A)), _ptr(tz), A, N, ne, R, d, _ptr(g_rep),
                                                 _stream()),
          "qmll_project_typed_backward")
    return g_rep


def project_typed_backward_sums(gx, sorted_slots, type_offsets, reductors, types, nslots, e_slots, B, n):
    """(g_rep [nslots,R] as `project_typed_backward` but with the rows of padded slots left unwritten,
    energies [B] = e_slots.view(B, n).sum(1)); one launch for small batches."""
    gx, reductors, e_slots = _f32(gx), _f32(reductors), _f32(e_slots)
    sorted_slots, type_offsets, types = _i32(sorted_slots), _i32(type_offsets), _i32(types).reshape(-1)
    ne, R, d = reductors.shape
    A, N = int(sorted_slots.shape[0]), int(nslots)
    if gx.shape[0] != A or gx.shape[1] != d or types.shape[0] != N or e_slots.numel() != B * n:
        raise RuntimeError("project_typed_backward_sums: gx %s for %d atoms, d=%d" % (tuple(gx.shape), A, d))
    g_rep = torch.empty((N, R), dtype=torch.float32, device=gx.device)
    energies = torch.empty(B, dtype=torch.float32, device=gx.device)
    check(_lib.lib().qmll_project_typed_backward_sums(_ptr(gx), _ptr(sorted_slots), _ptr(type_offsets), _ptr(reductors),
                                                      _ptr(_split_for(reductors, A)), _ptr(types), A, N, ne, R, d,
                                                      _ptr(g_rep), _ptr(e_slots), int(B), int(n), _ptr(energies),
                                                      _stream()),
          "qmll_project_typed_backward_sums")
    return g_rep, energies


def molecule_sums(e_slots, B, n):
    """energies [B] = sum over the n slots of each molecule of e_slots [B*n] (slots in ascending order:
    the same sums `project_typed_backward_sums` forms)."""
    e_slots = _f32(e_slots)
    if e_slots.numel() != B * n:
        raise RuntimeError("molecule_sums: %d slots for %d x %d" % (e_slots.numel(), B, n))
    energies = torch.empty(B, dtype=torch.float32, device=e_slots.device)
    check(_lib.lib().qmll_project_typed_backward_sums(None, None, None, None, None, None, 0, 0, 1, 1, 1, None,
                                                      _ptr(e_slots), int(B), int(n), _ptr(energies), _stream()),
          "qmll_project_typed_backward_sums")
    return energies


def _alpha32(alpha):
    """alpha in fp32; a model's fp64 alpha is converted once per tensor version, not per call."""
    if alpha.dtype == torch.float32:
        return alpha.contiguous()
    return presplit_cached(alpha, "f32", lambda t: t.float().contiguous())


def _zeroed_slots(e_zeroed, nslots, device):
    if e_zeroed is None:
        return torch.zeros(int(nslots), dtype=torch.float32, device=device)
    if e_zeroed.dtype != torch.float32 or e_zeroed.numel() != int(nslots) or not e_zeroed.is_contiguous():
        raise RuntimeError("e_zeroed must be a contiguous float32 tensor of %d entries" % int(nslots))
    return e_zeroed


def sorf_energy_sorted(x, type_offsets, sorted_slots, Dmat, bias, alpha, normalisation, ntransforms, nslots,
                       with_grad=True, e_zeroed=None):
    """Fused SORF + cos + energy on element-sorted rows x [A,d] -> (e_slots [nslots], gx [A,d] or None).
    e_zeroed: the caller's zero-filled f32 [nslots] to take the energies (else one is made here)."""
    x, Dmat, bias, alpha = _f32(x), _f32(Dmat), _f32(bias), _alpha32(alpha)
    type_offsets, sorted_slots = _i32(type_offsets), _i32(sorted_slots)
    ne, Tn, S, d = Dmat.shape
    A = int(sorted_slots.shape[0])
    if x.shape[0] != A or x.shape[1] != d or type_offsets.shape[0] != ne + 1:
        raise RuntimeError("sorf_energy_sorted: x is %s, expected [%d, %d]" % (tuple(x.shape), A, d))
    T = int(ntransforms)
    if T != Tn:
        raise RuntimeError("sorf_energy_sorted: %d diagonals stored per stack, %d transforms asked for" % (Tn, T))
    if tuple(bias.shape) != (ne, S * d) or alpha.numel() != S * d:
        raise RuntimeError("sorf_energy_sorted: bias %s / alpha with %d entries do not fit %d elements and %d features"
                           % (tuple(bias.shape), alpha.numel(), ne, S * d))
    e_slots = _zeroed_slots(e_zeroed, nslots, x.device)
    gx = torch.empty((A, d), dtype=torch.float32, device=x.device) if with_grad else None
    # the largest |bias|, a constant of the model, computed once per tensor version and left on the device
    bmax = presplit_cached(bias, "absmax", lambda t: t.abs().max().reshape(1))
    check(_lib.lib().qmll_sorf_energy_sorted(_ptr(x), _ptr(type_offsets), _ptr(sorted_slots), _ptr(Dmat), _ptr(bias),
                                             _ptr(alpha), _ptr(bmax), A, ne, d, S, T, float(normalisation), _ptr(e_slots),
                                             _ptr(gx), _stream()), "qmll_sorf_energy_sorted")
    return e_slots, gx


# ---------------------------------------------------------------------------------------
# RFF / Gram
# ---------------------------------------------------------------------------------------
def rff_features(x, W, b, mol_index, Zf):
    x, mol_index = _f32(x), _i32(mol_index)
    W, b = W.double().contiguous(), b.double().contiguous()
    A, d = x.shape
    F = W.shape[1]
    if W.shape[0] != d or b.numel() != F or mol_index.numel() != A or Zf.dtype != torch.float64 or Zf.shape[1] != F:
        raise RuntimeError("rff_features: x %s, W %s, b with %d entries, features %s do not fit together"
                           % (tuple(x.shape), tuple(W.shape), b.numel(), tuple(Zf.shape)))
    check(_lib.lib().qmll_rff_features(_ptr(x), _ptr(W), _ptr(b), _ptr(mol_index), A, d, F, int(Zf.shape[0]), _ptr(Zf),
                                       _stream()), "qmll_rff_features")
    return Zf


def rff_derivative_features(x, grad, W, b, mol_index, G, molecule_major=False):
    """molecule_major=True promises that mol_index is non-decreasing: the atomic-free
    matrix-core kernel is used (for d in 64/128/256)."""
    x, grad, mol_index = _f32(x), _f32(grad), _i32(mol_index)
    W, b = W.double().contiguous(), b.double().contiguous()
    A, n, _, d = grad.shape
    F = W.shape[1]
    if (tuple(x.shape) != (A, d) or W.shape[0] != d or b.numel() != F or mol_index.numel() != A
            or G.dtype != torch.float64 or tuple(G.shape[1:]) != (n, 3, F)):
        raise RuntimeError("rff_derivative_features: x %s, grad %s, W %s, b with %d entries, output %s do not fit together"
                           % (tuple(x.shape), tuple(grad.shape), tuple(W.shape), b.numel(), tuple(G.shape)))
    nmol = int(G.shape[0])
    seg = None
    if molecule_major:
        bounds = torch.arange(nmol + 1, dtype=torch.int32, device=x.device)
        seg = torch.searchsorted(mol_index, bounds).to(torch.int32)
    check(_lib.lib().qmll_rff_derivative_features(_ptr(x), _ptr(grad), _ptr(W), _ptr(b), _ptr(mol_index), _ptr(seg), A, n,
                                                  d, F, nmol, _ptr(G), _stream()), "qmll_rff_derivative_features")
    return G


_PRESPLIT = {}    # (id(tensor), kind) -> (weak reference, version, address, prepared buffer)


def _version(t):
    try:
        return t._version
    except RuntimeError:      # inference tensors keep no version counter
        return -1


def presplit_cached(t, kind, make):
    """The prepared (pre-split) form of a model constant `t`, made once by `make(t)` and reused until
    the tensor object dies, is written to in place (its version counter moves) or changes its storage."""
    key = (id(t), kind)
    hit = _PRESPLIT.get(key)
    if hit is not None and hit[0]() is t and hit[1] == _version(t) and hit[2] == t.data_ptr():
        return hit[3]
    buf = make(t)
    _PRESPLIT[key] = (weakref.ref(t, lambda _r, k=key: _PRESPLIT.pop(k, None)), _version(t), t.data_ptr(), buf)
    return buf


def rff_presplit(W):
    """W f32 [ne,d,F] in the form the fused RFF predict kernel multiplies with (qmll_rff_presplit):
    an opaque uint8 device buffer."""
    W = _f32(W)
    ne, d, F = W.shape
    nbytes = int(_lib.lib().qmll_rff_presplit_bytes(ne, d, F))
    if nbytes == 0:
        raise RuntimeError("rff_presplit: the fused kernel exists for d = 64 or 128 and a multiple of 32 features, "
                           "not d = %d, F = %d" % (d, F))
    out = torch.empty(nbytes, dtype=torch.uint8, device=W.device)
    check(_lib.lib().qmll_rff_presplit(_ptr(W), ne, d, F, _ptr(out), nbytes, _stream()), "qmll_rff_presplit")
    return out


def rff_energy_sorted(x, type_offsets, sorted_slots, W, b, alpha, nslots, with_grad=True, e_zeroed=None):
    """Fused RFF energy (and gradient) on element-sorted rows x [A,d]; W [ne,d,F], b [ne,F],
    alpha [F] fp32 -> (e_slots [nslots], gx [A,d] or None).  W is split for the kernel on its first
    use and the split form kept until W changes.  e_zeroed: as for sorf_energy_sorted."""
    x, W, b, alpha = _f32(x), _f32(W), _f32(b), _alpha32(alpha)
    type_offsets, sorted_slots = _i32(type_offsets), _i32(sorted_slots)
    ne, d, F = W.shape
    A = int(sorted_slots.shape[0])
    if x.shape[0] != A or x.shape[1] != d or type_offsets.shape[0] != ne + 1 or b.shape[0] != ne or b.shape[1] != F:
        raise RuntimeError("rff_energy_sorted: x %s, W %s, b %s do not fit together"
                           % (tuple(x.shape), tuple(W.shape), tuple(b.shape)))
    if alpha.numel() != F:
        raise RuntimeError("rff_energy_sorted: alpha has %d entries for %d features" % (alpha.numel(), F))
    Wsplit = presplit_cached(W, "rff", rff_presplit)
    e_slots = _zeroed_slots(e_zeroed, nslots, x.device)
    gx = torch.empty((A, d), dtype=torch.float32, device=x.device) if with_grad else None
    check(_lib.lib().qmll_rff_energy_sorted(_ptr(x), _ptr(type_offsets), _ptr(sorted_slots), _ptr(Wsplit), _ptr(b),
                                            _ptr(alpha), A, ne, d, F, _ptr(e_slots), _ptr(gx), _stream()),
          "qmll_rff_energy_sorted")
    return e_slots, gx


def cholesky_solve_spd(A, b, overwrite_a=False):
    """x = A^-1 b for a symmetric positive definite fp64 A [F,F] and b [F] or [F,1], by the
    in-place upper Cholesky factorisation of the library.  Only the upper triangle of A is read.
    Returns (x, info): info is a device int32 tensor, 0 on success, else 1 + the index of the first
    non-positive pivot, or -1 if a bounded wait inside the library ran out (never seen); x is then
    meaningless.  A is destroyed when overwrite_a is True."""
    if A.dtype != torch.float64 or A.dim() != 2 or A.shape[0] != A.shape[1] or A.stride(1) != 1:
        raise RuntimeError("cholesky_solve_spd needs a square float64 matrix with contiguous rows")
    F = int(A.shape[0])
    if b.dtype != torch.float64 or b.numel() != F:
        raise RuntimeError("cholesky_solve_spd: b must hold F float64 values")
    U = A if overwrite_a else A.clone()
    ld = int(U.stride(0))
    if ld % 2 != 0:
        raise RuntimeError("cholesky_solve_spd: the row stride must be even")
    L = _lib.lib()
    work = torch.empty(int(L.qmll_cholesky_workspace_bytes(F)) // 8 + 1, dtype=torch.float64, device=A.device)
    info = torch.zeros(1, dtype=torch.int32, device=A.device)
    x = b.detach().clone().contiguous()
    check(L.qmll_cholesky_f64(_ptr(U), F, ld, _ptr(work), _ptr(info), _stream()), "qmll_cholesky_f64")
    check(L.qmll_cholesky_solve_f64(_ptr(U), F, ld, _ptr(work), _ptr(x), _stream()), "qmll_cholesky_solve_f64")
    return x, info


def gram_mirror(ZTZ):
    """Copy the upper triangle of ZTZ onto the lower one (after `gram(..., mirror=False)` calls)."""
    if ZTZ.dtype != torch.float64 or not ZTZ.is_contiguous() or ZTZ.shape[0] != ZTZ.shape[1]:
        raise RuntimeError("gram_mirror needs a contiguous square float64 matrix")
    check(_lib.lib().qmll_gram_mirror_f64(_ptr(ZTZ), int(ZTZ.shape[0]), _stream()), "qmll_gram_mirror_f64")
    return ZTZ


_GRAM_WS = {}


def _gram_workspace(device):
    """The Gram kernel's workspace for the split last round of tiles: one buffer per device and
    stream, kept between calls (calls on one stream are ordered; calls that may overlap on a device
    must not share a workspace)."""
    key = (device.index if device.index is not None else torch.cuda.current_device(), _stream().value)
    ws = _GRAM_WS.get(key)
    if ws is None:
        ws = torch.empty(int(_lib.lib().qmll_gram_workspace_bytes()) // 8, dtype=torch.float64, device=device)
        _GRAM_WS[key] = ws
    return ws


def gram(Zrows, y, ZTZ, ZTy, f0=None, f1=None, mirror=True):
    """ZTZ += Z^T Z (or the row block f0:f1 of it), ZTy += Z^T y, fp64, in place.
    mirror=False (full matrix only) accumulates just the tiles on or above the diagonal: a
    caller adding several batches finishes with one `gram_mirror(ZTZ)`."""
    if Zrows.dtype != torch.float64 or not Zrows.is_contiguous():
        raise RuntimeError("gram needs a contiguous float64 row matrix")
    M, F = Zrows.shape
    yv = None
    if y is not None:
        yv = y.reshape(-1).double().contiguous()
        if yv.shape[0] != M:
            raise RuntimeError("targets have %d rows, features have %d" % (yv.shape[0], M))
    zty = ZTy if ZTy is not None else None
    if f0 is None:
        # with a workspace the last, sparsely filled round of tiles is split over the idle CUs
        ws = _gram_workspace(Zrows.device) if M >= 2048 else None
        check(_lib.lib().qmll_gram_upper_ws_f64(_ptr(Zrows), _ptr(yv), M, F, _ptr(ZTZ), _ptr(zty), _ptr(ws),
                                                ws.numel() * 8 if ws is not None else 0, _stream()),
              "qmll_gram_upper_ws_f64")
        if mirror:
            check(_lib.lib().qmll_gram_mirror_f64(_ptr(ZTZ), F, _stream()), "qmll_gram_mirror_f64")
    else:
        check(_lib.lib().qmll_gram_tile_f64(_ptr(Zrows), _ptr(yv), M, F, int(f0), int(f1), _ptr(ZTZ), _ptr(zty),
                                            _stream()), "qmll_gram_tile_f64")
    return ZTZ, ZTy


def matmul_and_reduce(A, B, C):
    A, B = _f32(A), _f32(B)
    if C.dtype != torch.float64 or not C.is_contiguous():
        raise RuntimeError("matmul_and_reduce accumulates into a contiguous float64 tensor")
    check(_lib.lib().qmll_matmul_and_reduce(_ptr(A), _ptr(B), A.shape[0], A.shape[1], B.shape[1], _ptr(C), _stream()),
          "qmll_matmul_and_reduce")
    return C


# ---------------------------------------------------------------------------------------
# torch.ops registration (names and argument order of the reference's TORCH_LIBRARY blocks)
# ---------------------------------------------------------------------------------------
_FCHL_SIG = ("Tensor X, Tensor Z, Tensor species, Tensor atomIDs, Tensor molIDs, Tensor atom_counts, Tensor cell, "
             "Tensor inv_cell, Tensor Rs2, Tensor Rs3, Tensor eta2, Tensor eta3, Tensor two_body_decay, "
             "Tensor three_body_weight, Tensor three_body_decay, Tensor rcut")

_registered = False
_libs = []
TORCH_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libqmll_torch.so")
OPS_BACKEND = None   # "c++" (libqmll_torch.so) or "python" (the torch.library definitions below)


def _fchl_fwd_impl(X, Z, species, atomIDs, molIDs, atom_counts, cell, inv_cell, Rs2, Rs3, eta2, eta3, two_body_decay,
                   three_body_weight, three_body_decay, rcut):
    for t, name in ((X, "coordinates"), (Z, "charges"), (species, "species"), (atomIDs, "atomIDs"),
                    (molIDs, "molIDs"), (atom_counts, "atom_counts"), (cell, "cell"), (inv_cell, "inv_cell")):
        _need_cuda(t, name)                                  # torchscript/FCHL19.cpp:251-258
    prm = make_params(species.shape[0], Rs2, Rs3, eta2, eta3, two_body_decay, three_body_weight, three_body_decay, rcut)
    types = element_types(X, Z, atom_counts, species)
    return fchl_forward(X, types, cell, inv_cell, atomIDs, molIDs, atom_counts, Rs2, Rs3, prm)


def _fchl_bwd_impl(grad, X, Z, species, atomIDs, molIDs, atom_counts, cell, inv_cell, Rs2, Rs3, eta2, eta3,
                   two_body_decay, three_body_weight, three_body_decay, rcut):
    prm = make_params(species.shape[0], Rs2, Rs3, eta2, eta3, two_body_decay, three_body_weight, three_body_decay, rcut)
    types = element_types(X, Z, atom_counts, species)
    g = fchl_vjp(grad, X, types, cell, inv_cell, atomIDs, molIDs, atom_counts, Rs2, Rs3, prm)
    return g.reshape(X.shape)


def _fchl_and_derivative_impl(X, Z, species, atomIDs, molIDs, atom_counts, cell, inv_cell, Rs2, Rs3, eta2, eta3,
                              two_body_decay, three_body_weight, three_body_decay, rcut, gradients):
    prm = make_params(species.shape[0], Rs2, Rs3, eta2, eta3, two_body_decay, three_body_weight, three_body_decay, rcut)
    types = element_types(X, Z, atom_counts, species)
    if gradients:
        rep, jac = fchl_jacobian(X, types, cell, inv_cell, atomIDs, molIDs, atom_counts, Rs2, Rs3, prm)
        return [rep, jac]
    return [fchl_forward(X, types, cell, inv_cell, atomIDs, molIDs, atom_counts, Rs2, Rs3, prm)]


def register_ops():
    """Define qml_lightning_fchl::* and qml_lightning_sorf::* once per process."""
    global _registered, OPS_BACKEND
    if _registered:
        return
    _registered = True
    # The operators live in libqmll_torch.so (TORCH_LIBRARY from C++, as in the reference: low
    # dispatch cost, usable by hosts without Python).  The definitions below do the same from
    # Python over the same kernels; they serve when that library has not been built, when
    # QML_LIGHTNING_AMD_PY_OPS=1 asks for them, or when QML_LIGHTNING_AMD_LIB points to another
    # copy of libqmll.so (the C++ library is linked to the copy beside it).
    want_python = os.environ.get("QML_LIGHTNING_AMD_PY_OPS") == "1" or "QML_LIGHTNING_AMD_LIB" in os.environ
    if not want_python and os.path.exists(TORCH_LIB_PATH) and os.path.exists(_lib.LIB_PATH):
        torch.ops.load_library(TORCH_LIB_PATH)
        OPS_BACKEND = "c++"
        return
    OPS_BACKEND = "python"
    Library = torch.library.Library

    fl = Library("qml_lightning_fchl", "DEF")
    fl.define("fchl_forwards(%s) -> Tensor" % _FCHL_SIG)
    fl.define("fchl_backwards(Tensor grad, %s) -> Tensor" % _FCHL_SIG)
    fl.define("get_fchl_and_derivative(%s, bool gradients) -> Tensor[]" % _FCHL_SIG)
    fl.define("get_element_types(Tensor coordinates, Tensor charges, Tensor natom_counts, Tensor species) -> Tensor")
    fl.define("get_num_neighbours(Tensor coordinates, Tensor natoms, Tensor rcut, Tensor lattice_vecs, "
              "Tensor inv_lattice_vecs) -> Tensor")
    fl.define("get_neighbour_list(Tensor coordinates, Tensor natoms, Tensor max_neighbours, Tensor rcut, "
              "Tensor lattice_vecs, Tensor inv_lattice_vecs) -> Tensor")
    fl.impl("fchl_forwards", _fchl_fwd_impl, "CompositeExplicitAutograd")
    fl.impl("fchl_backwards", _fchl_bwd_impl, "CompositeExplicitAutograd")
    fl.impl("get_fchl_and_derivative", _fchl_and_derivative_impl, "CompositeExplicitAutograd")
    fl.impl("get_element_types", lambda X, Z, n, s: element_types(X, Z, n, s), "CompositeExplicitAutograd")
    fl.impl("get_num_neighbours", lambda X, n, rc, c, ic: num_neighbours(X, n, rc, c, ic), "CompositeExplicitAutograd")
    fl.impl("get_neighbour_list", lambda X, n, mx, rc, c, ic: neighbour_list(X, n, mx, rc, c, ic), "CompositeExplicitAutograd")

    def fchl_setup(ctx, inputs, output):
        ctx.save_for_backward(*inputs)

    def fchl_backward(ctx, grad):
        # autograd on X only (torchscript/FCHL19.cpp:314)
        g = torch.ops.qml_lightning_fchl.fchl_backwards(grad.contiguous(), *ctx.saved_tensors)
        return (g,) + (None,) * 15

    torch.library.register_autograd("qml_lightning_fchl::fchl_forwards", fchl_backward, setup_context=fchl_setup,
                                    lib=fl)

    sl = Library("qml_lightning_sorf", "DEF")
    sl.define("get_SORF_coefficients(Tensor u, Tensor d, Tensor coeff_normalisation, Tensor ntransforms) -> Tensor")
    sl.define("get_SORF_coefficients_backward(Tensor grad, Tensor d, Tensor coeff_normalisation, Tensor ntransforms) "
              "-> Tensor")
    sl.define("get_cos_features(Tensor coeffs, Tensor b, Tensor nmol, Tensor batch_indexes) -> Tensor")
    sl.define("get_cos_features_backward(Tensor grad, Tensor coeffs, Tensor b, Tensor nmol, Tensor batch_indexes) "
              "-> Tensor")
    sl.impl("get_SORF_coefficients",
            lambda u, d, cn, nt: sorf_forward(u, d, _scalar(cn), int(nt.item())), "CompositeExplicitAutograd")   # SORF.cpp:85
    sl.impl("get_SORF_coefficients_backward",
            lambda g, d, cn, nt: sorf_adjoint(g, d, _scalar(cn), int(nt.item())), "CompositeExplicitAutograd")   # SORF.cpp:99
    sl.impl("get_cos_features",
            lambda c, b, nmol, idx: cos_features(c, b, int(nmol.item()), idx), "CompositeExplicitAutograd")      # SORF.cpp:118
    sl.impl("get_cos_features_backward",
            lambda g, c, b, nmol, idx: cos_features_backward(g, c, b, int(nmol.item()), idx), "CompositeExplicitAutograd")

    def sorf_setup(ctx, inputs, output):
        _, d, cn, nt = inputs
        ctx.save_for_backward(d, cn, nt)

    def sorf_backward(ctx, grad):
        d, cn, nt = ctx.saved_tensors
        return torch.ops.qml_lightning_sorf.get_SORF_coefficients_backward(grad.contiguous(), d, cn, nt), None, None, None

    def cos_setup(ctx, inputs, output):
        ctx.save_for_backward(*inputs)

    def cos_backward(ctx, grad):
        c, b, nmol, idx = ctx.saved_tensors
        return torch.ops.qml_lightning_sorf.get_cos_features_backward(grad.contiguous(), c, b, nmol, idx), None, None, None

    torch.library.register_autograd("qml_lightning_sorf::get_SORF_coefficients", sorf_backward,
                                    setup_context=sorf_setup, lib=sl)
    torch.library.register_autograd("qml_lightning_sorf::get_cos_features", cos_backward, setup_context=cos_setup,
                                    lib=sl)
    _libs.extend([fl, sl])
