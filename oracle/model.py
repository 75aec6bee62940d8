"""CPU oracle (test infrastructure, never the product path): the whole predict and
training-row pipeline in fp64, chained from oracle.fchl19 and oracle.sorf.

Follows (paths relative to the reference tree):
  * TorchScript forward ............ qml_lightning/models/hadamard_features.py:82-123
  * forces by autograd ............. qml_lightning/models/hadamard_features.py:156-162 with the
                                     backward formulas of qml_lightning/cuda/torchscript/SORF.cpp:89-135
                                     and qml_lightning/cuda/torchscript/FCHL19.cpp:279-315
  * RFF forward .................... qml_lightning/models/random_features.py:69-102
  * training rows .................. qml_lightning/models/kernel.py:93-192

Pinned by the reference's aspirin known-answer vector (energy + forces) and by the
agreement of its two independent routes (G.alpha == -dE/dX); see tests/test_oracle_kat.py.
"""
import numpy as np

from . import fchl19, sorf


def format_batch(coords, charges):
    """Zero-padded batch the way format_data lays it out (kernel.py:630-695)."""
    B = len(coords)
    natoms = np.array([len(c) for c in coords], dtype=np.int32)
    n = int(natoms.max())
    X = np.zeros((B, n, 3))
    Z = np.zeros((B, n))
    atomIDs, molIDs = [], []
    for m in range(B):
        X[m, :natoms[m]] = coords[m]
        Z[m, :natoms[m]] = charges[m]
        atomIDs += list(range(natoms[m]))
        molIDs += [m] * int(natoms[m])
    return X, Z, np.array(atomIDs, dtype=np.int32), np.array(molIDs, dtype=np.int32), natoms


def representation(X, Z, atomIDs, molIDs, natoms, prm, cell=None, inv_cell=None, jacobian=False):
    nneigh, nlist = fchl19.neighbours(X, natoms, prm.rcut, cell, inv_cell)
    types = fchl19.element_types(Z, natoms, prm.species)
    rep = fchl19.forward(X, types, atomIDs, molIDs, nlist, nneigh, prm, cell, inv_cell)
    ctx = (types, nlist, nneigh)
    if jacobian:
        J = fchl19.jacobian(X, types, atomIDs, molIDs, nlist, nneigh, prm, cell, inv_cell)
        return rep, J, ctx
    return rep, ctx


def sorf_energy_forces(X, Z, atomIDs, molIDs, natoms, prm, elements, reductors, Dmat, bias, alpha,
                       sigma, forces=True, cell=None, inv_cell=None):
    """E [B] and F = -dE/dX [B,n,3] by the reverse-mode route of the TorchScript model."""
    X = np.asarray(X, dtype=np.float64)
    B, n, _ = X.shape
    rep, (types, nlist, nneigh) = representation(X, Z, atomIDs, molIDs, natoms, prm, cell, inv_cell)
    T, S, d = np.asarray(Dmat[0]).shape
    F = S * d
    norm = np.sqrt(d) / sigma
    q = np.asarray(Z).astype(np.int64)
    alpha = np.asarray(alpha, dtype=np.float64)
    Zfeat = np.zeros((B, F))
    saved = []
    for ei, e in enumerate(elements):
        mask = q == int(e)
        if not mask.any():
            continue
        mol_index = np.nonzero(mask)[0]
        sub = sorf.project(rep[mask], reductors[ei])
        coeffs = sorf.sorf_coefficients(sub, Dmat[ei], norm).reshape(len(sub), F)
        Zfeat += sorf.cos_features(coeffs, bias[ei], mol_index, B)
        saved.append((ei, mask, mol_index, coeffs))
    E = Zfeat @ alpha
    if not forces:
        return E, None, Zfeat
    # d(-sum E)/dZfeat = -alpha for every molecule
    gZ = -np.repeat(alpha[None, :], B, axis=0)
    grep = np.zeros_like(rep)
    for ei, mask, mol_index, coeffs in saved:
        gc = sorf.cos_features_backward(gZ, coeffs, bias[ei], mol_index)
        gsub = sorf.sorf_adjoint(gc.reshape(len(coeffs), S, d), Dmat[ei], norm)
        grep[mask] = gsub @ np.asarray(reductors[ei], dtype=np.float64).T
    Fout = fchl19.vjp(grep, X, types, atomIDs, molIDs, nlist, nneigh, prm, cell, inv_cell)
    return E, Fout, Zfeat


def rff_energy_forces(X, Z, atomIDs, molIDs, natoms, prm, elements, reductors, W, b, alpha,
                      forces=True):
    """RFF twin of sorf_energy_forces (random_features.py:82-102)."""
    X = np.asarray(X, dtype=np.float64)
    B, n, _ = X.shape
    rep, (types, nlist, nneigh) = representation(X, Z, atomIDs, molIDs, natoms, prm)
    F = np.asarray(W[0]).shape[1]
    q = np.asarray(Z).astype(np.int64)
    alpha = np.asarray(alpha, dtype=np.float64)
    Zfeat = np.zeros((B, F))
    saved = []
    for ei, e in enumerate(elements):
        mask = q == int(e)
        if not mask.any():
            continue
        mol_index = np.nonzero(mask)[0]
        sub = sorf.project(rep[mask], reductors[ei])
        Zfeat += sorf.rff_features(sub, W[ei], b[ei], mol_index, B)
        saved.append((ei, mask, mol_index, sub))
    E = Zfeat @ alpha
    if not forces:
        return E, None, Zfeat
    grep = np.zeros_like(rep)
    nf = np.sqrt(2.0 / F)
    for ei, mask, mol_index, sub in saved:
        We = np.asarray(W[ei], dtype=np.float64)
        arg = sub @ We + np.asarray(b[ei], dtype=np.float64)[None, :]
        garg = -alpha[None, :] * (-np.sin(arg)) * nf          # d(-E)/d arg
        grep[mask] = (garg @ We.T) @ np.asarray(reductors[ei], dtype=np.float64).T
    Fout = fchl19.vjp(grep, X, types, atomIDs, molIDs, nlist, nneigh, prm)
    return E, Fout, Zfeat


def sorf_training_rows(X, Z, atomIDs, molIDs, natoms, prm, elements, reductors, Dmat, bias, sigma,
                       E=None, F=None):
    """Rows [M,F] and targets [M,1] of one training batch (kernel.py:105-170)."""
    if F is not None:
        rep, J, _ = representation(X, Z, atomIDs, molIDs, natoms, prm, jacobian=True)
    else:
        rep, _ = representation(X, Z, atomIDs, molIDs, natoms, prm)
        J = None
    Zf, G = sorf.hadamard_model_features(rep, Z, elements, reductors, Dmat, bias, sigma, jac=J)
    return sorf.training_rows(Zf, G, E, F)
