"""PCA projection of representations and their Jacobians
(qml_lightning/representations/dimensionality_reduction.py:47-72): plain dense GEMMs, run
by the BLAS library."""
import torch


def project_representation(X, reductor):
    """[nsamples, repsize] @ [repsize, npcas]."""
    return torch.matmul(X, reductor)


def project_derivative(dX, reductor):
    """[nsamples, natoms, 3, repsize] -> [nsamples, natoms, 3, npcas]."""
    return torch.matmul(dX, reductor)
