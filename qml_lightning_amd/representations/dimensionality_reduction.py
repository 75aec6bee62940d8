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


def get_reductors(gto, charges, npcas, species):
    """{element: [repsize, npcas]}: leading left singular vectors of up to 512 randomly chosen
    representation rows of each element (dimensionality_reduction.py:13-44).  gto [..., repsize],
    charges of the same leading shape."""
    out = {}
    for e in species:
        rows = gto[charges == e]
        if rows.shape[0] == 0:
            continue
        pick = torch.randperm(rows.size(0), device=rows.device)[:512]
        U, sv, _ = torch.linalg.svd(rows[pick].T, full_matrices=False)
        kept = 100 - (sv.sum() - sv[:npcas].sum()) / sv.sum() * 100
        red = U[:, :npcas]
        print(f"{red.shape[0]} -> {red.shape[1]}  Cumulative Explained Feature Variance = {float(kept):6.2f} %%")
        out[e] = red
    return out
