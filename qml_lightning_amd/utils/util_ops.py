"""Free-function forms of the model's data helpers (qml_lightning/utils/util_ops.py:10-213): the
per-element self-energy fit and the list -> padded-tensor formatting that the reference's own
unit tests call without building a model.  The model methods (models/kernel.py) carry the
unit-conversion and self-energy options; these do not, as in the reference."""
import numpy as np
import torch


def _device():
    return torch.device("cuda:0")


def calculate_self_energy(Q, E, elements):
    """Least-squares energy per element from composition counts (util_ops.py:10-53): returns
    fp64 [max(elements) + 1], zero for elements that are not listed."""
    elements = torch.as_tensor(elements)
    counts = np.zeros((len(Q), len(elements)), dtype=np.float64)
    for i, q in enumerate(Q):
        q = np.asarray(q)
        for j, e in enumerate(elements):
            counts[i, j] = np.count_nonzero(q == int(e))
    X = torch.from_numpy(counts)
    y = torch.as_tensor(np.asarray(E, dtype=np.float64))[:, None]
    beta = torch.linalg.lstsq(X.T @ X, X.T @ y).solution[:, 0]
    species = elements.long()
    self_energy = torch.zeros(int(species.max()) + 1, dtype=torch.float64)
    self_energy[species] = beta
    return self_energy


def format_data(X, Q, E=None, F=None, cells=None, inv_cells=None, same_mol=False):
    """Per-molecule arrays -> zero-padded device tensors 'coordinates' f32 [B,n,3], 'charges' f32
    [B,n], 'natom_counts' / 'atomIDs' / 'molIDs' i32, 'energies' f64, 'forces', 'cells' /
    'inv_cells' f32 ([0,3,3] when there is no cell) (util_ops.py:56-213).  A single molecule
    (2-D X, 1-D Q) counts as a batch of one.  same_mol: X [B,n,3] and Q [B,n] are whole arrays of
    one composition, uploaded as they are (forces then stay fp32 and absent targets add no key,
    as in the reference)."""
    dev = _device()
    if isinstance(X, np.ndarray) and X.ndim == 2:
        X = X[None]
    if isinstance(Q, np.ndarray) and Q.ndim == 1:
        Q = Q[None]
    if isinstance(F, np.ndarray) and F.ndim == 2:
        F = F[None]
    if isinstance(cells, np.ndarray) and cells.ndim == 2:
        cells, inv_cells = cells[None], np.asarray(inv_cells)[None]
    B = len(X)
    none = torch.empty((0, 3, 3), device=dev)
    data = {}
    if same_mol:
        coords = torch.as_tensor(np.asarray(X)).float().to(dev)
        n = coords.shape[1]
        data['coordinates'] = coords
        data['charges'] = torch.as_tensor(np.asarray(Q)).float().to(dev)
        data['natom_counts'] = torch.full((B,), n, dtype=torch.int32, device=dev)
        data['atomIDs'] = torch.arange(n, dtype=torch.int32, device=dev).repeat(B)
        data['molIDs'] = torch.arange(B, dtype=torch.int32, device=dev).repeat_interleave(n)
        if E is not None:
            data['energies'] = torch.as_tensor(np.asarray(E)).double().to(dev)
        if F is not None:
            data['forces'] = torch.as_tensor(np.asarray(F)).float().to(dev)
    else:
        counts = np.fromiter((len(x) for x in X), dtype=np.int32, count=B)
        n = int(counts.max()) if B else 0
        molIDs = np.repeat(np.arange(B, dtype=np.int32), counts)
        atomIDs = (np.arange(int(counts.sum())) - np.repeat(np.cumsum(counts) - counts, counts)).astype(np.int32)
        flat = molIDs.astype(np.int64) * n + atomIDs
        coords = np.zeros((B, n, 3), dtype=np.float32)
        charges = np.zeros((B, n), dtype=np.float32)
        if B:
            coords.reshape(-1, 3)[flat] = np.concatenate([np.asarray(x, dtype=np.float32).reshape(-1, 3) for x in X])
            charges.reshape(-1)[flat] = np.concatenate([np.asarray(q, dtype=np.float32).reshape(-1) for q in Q])
        data['coordinates'] = torch.from_numpy(coords).to(dev)
        data['charges'] = torch.from_numpy(charges).to(dev)
        data['natom_counts'] = torch.from_numpy(counts).to(dev)
        data['atomIDs'] = torch.from_numpy(atomIDs).to(dev)
        data['molIDs'] = torch.from_numpy(molIDs).to(dev)
        data['energies'] = None
        data['forces'] = None
        if E is not None:
            data['energies'] = torch.from_numpy(np.asarray(E, dtype=np.float64).reshape(B).copy()).to(dev)
        if F is not None:
            forces = np.zeros((B, n, 3), dtype=np.float64)
            if B:
                forces.reshape(-1, 3)[flat] = np.concatenate([np.asarray(f, dtype=np.float64).reshape(-1, 3) for f in F])
            data['forces'] = torch.from_numpy(forces).to(dev)
    data['cells'], data['inv_cells'] = none, none
    if cells is not None:
        data['cells'] = torch.from_numpy(np.asarray(cells, dtype=np.float32).reshape(B, 3, 3)).to(dev)
        data['inv_cells'] = torch.from_numpy(np.asarray(inv_cells, dtype=np.float32).reshape(B, 3, 3)).to(dev)
    return data
