"""BaseKernel: host orchestration shared by the SORF and RFF models
(qml_lightning/models/kernel.py:15-722 of the reference): batch formatting, the training
loop that assembles the rows Z = [Z_E ; G] and accumulates Z^T Z / Z^T y, the solve, the
explicit-Jacobian predict route, reductor fitting and self energies.

Same class / method names, argument meaning, row order and dtypes as the reference; what
differs is underneath: one fp64 row buffer per batch (energy rows and force rows are
views of it, no concatenation copy), per-element atom indices built once on the host by
`format_data` (no boolean-mask device syncs), the hand-written fp64 MFMA Gram kernel, and
no `empty_cache()` between batches.
"""
import weakref

import numpy as np
import torch

from .. import ops
from ..cuda.utils_gpu import matmul_and_reduce


def _default_device():
    return torch.device("cuda" if torch.cuda.is_available() else "cpu")


_ALPHA32 = weakref.WeakKeyDictionary()    # model -> (alpha it was made from, its version, fp32 copy)


def alpha_f32(model):
    """model.alpha as fp32 (what the predict routes contract with), converted once per value of
    alpha instead of once per call: one launch less per step, which counts for single molecules."""
    a = model.alpha
    if a.dtype == torch.float32:
        return a
    hit = _ALPHA32.get(model)
    if hit is None or hit[0] is not a or hit[1] != a._version:
        hit = (a, a._version, a.float())
        _ALPHA32[model] = hit
    return hit[2]


def rep_from_attribute_tree(tree):
    """An FCHLCuda with exactly the tensors a saved model's `rep` sub-module holds (attribute
    names and dtypes of qml_lightning/representations/FCHL.py:21-46): the radial grids, the
    weight with sqrt(eta3/pi) already folded in and the fp32 scalars are taken as stored, not
    recomputed from rounded hyper-parameters."""
    from ..representations.FCHL import FCHLCuda
    if not str(tree.get("__class__", "")).endswith("FCHLCuda"):
        raise ValueError("model file: the representation is %r, only FCHLCuda is supported" % tree.get("__class__"))
    species = np.asarray(tree["species"])
    rep = FCHLCuda(species=species.astype(np.int64), rcut=float(tree["rcut"]), nRs2=int(tree["nRs2"]),
                   nRs3=int(tree["nRs3"]), eta2=float(tree["eta2"]), eta3=float(tree["eta3"]),
                   two_body_decay=float(tree["two_body_decay"]), three_body_weight=1.0,
                   three_body_decay=float(tree["three_body_decay"]))
    dev = rep.device
    rep.species = torch.from_numpy(species.astype(np.float32)).to(dev)
    for name in ("rcut", "eta2", "eta3", "two_body_decay", "three_body_weight", "three_body_decay"):
        setattr(rep, name, torch.from_numpy(np.asarray(tree[name], dtype=np.float32).reshape(())).clone())
    rep.nRs2 = torch.tensor(int(tree["nRs2"]))
    rep.nRs3 = torch.tensor(int(tree["nRs3"]))
    rep.Rs2 = torch.from_numpy(np.asarray(tree["Rs2"], dtype=np.float32)).to(dev)
    rep.Rs3 = torch.from_numpy(np.asarray(tree["Rs3"], dtype=np.float32)).to(dev)
    if int(tree["fp_size"]) != rep.fp_size:
        raise ValueError("model file: fp_size %d does not follow from its species and grids (%d)"
                         % (int(tree["fp_size"]), rep.fp_size))
    return rep


class BaseKernel():

    def __init__(self, rep, npcas, elements, sigma, llambda):
        super(BaseKernel, self).__init__()
        self.npcas = npcas
        self.self_energy = None
        self.elements = torch.tensor(np.asarray(elements))
        self.rep = rep
        dev = _default_device()
        self.reductors = torch.zeros(len(elements), rep.get_repsize(), npcas, dtype=torch.float32, device=dev)
        self.element2index = torch.zeros(int(max(elements)) + 1, dtype=torch.long)
        for i, e in enumerate(self.elements):
            self.element2index[int(e)] = i
        self._convert_from_hartree_to_kcal = False
        self.hartree2kcalmol = 627.5
        self._subtract_self_energies = False
        self.sigma = sigma
        self.llambda = llambda
        self._queue_force_rows = False

    # -- to be provided by the feature model -------------------------------------------
    def finish_features(self, derivative_matrix=None, overwrite=False):
        """Called once per batch after the loop over elements; models that queue work in
        calculate_features run it here."""
        return None

    def writes_force_rows(self):
        """True when finish_features writes every element of the force-feature block itself
        (overwrite=True), so that the block need not be cleared first."""
        return False

    def calculate_features(self, rep, element, indexes, feature_matrix, grad=None, derivative_matrix=None):
        raise NotImplementedError("Abstract method only.")

    def nfeatures(self):
        raise NotImplementedError("Abstract method only.")

    def predict(self, X, Q, max_natoms, cells=None, inv_cells=None, forces=False, print_info=True, use_backward=True):
        raise NotImplementedError("Abstract method only.")

    # -- rows of one batch ----------------------------------------------------------------
    def _batch_projected(self, data, with_forces):
        """Everything of a formatted batch that does not depend on sigma: per element the projected
        representation rows [A_e, npcas] (and projected Jacobian rows [A_e, n, 3, npcas]) with the
        molecule index of each row (kernel.py:141-160 up to the call of calculate_features)."""
        coordinates, charges = data['coordinates'], data['charges']
        atomIDs, molIDs, natom_counts = data['atomIDs'], data['molIDs'], data['natom_counts']
        cells, inv_cells = data['cells'], data['inv_cells']
        B, n = charges.shape
        if with_forces:
            representation, rep_derivative = self.rep.get_representation_and_derivative(
                coordinates, charges, atomIDs, molIDs, natom_counts, cells, inv_cells)
        else:
            representation = self.rep.get_representation(coordinates, charges, atomIDs, molIDs, natom_counts, cells,
                                                         inv_cells)
            rep_derivative = None
        flat_rep = representation.view(B * n, -1)
        # the atoms of every element, element after element in the order of the projection matrices:
        # one typed product then serves all elements (for the derivative rows, 3n rows per atom), where
        # the reference copies each element's rows out and multiplies them one element at a time
        ne = self.reductors.shape[0]
        items = []
        ecounts = data.get('element_counts')
        if ecounts is not None:
            # the element-sorted atom index is built on the device (one counting sort over the batch,
            # stable: ascending slot within an element, the order of `rep[Z == e]`); only the per-element
            # counts, which the formatter took from the host copy of the charges, are needed here
            counts = [0] * ne
            order = [None] * ne
            for e in self.elements:
                t = int(self.element2index[int(e)])
                counts[t], order[t] = int(ecounts.get(int(e), 0)), e
            offsets = np.concatenate(([0], np.cumsum(counts))).astype(np.int32)
            if offsets[-1] > 0:
                types = ops.element_types(coordinates, charges, natom_counts, self._sort_species_tensor())
                slots, type_offsets = ops.sort_atoms_by_type(types, atomIDs, molIDs, n, ne)
                slots = slots[:int(offsets[-1])]
        else:
            lists = [None] * ne
            for e in self.elements:
                lists[self.element2index[int(e)]] = (e, self._element_index(data, charges, int(e)))
            counts = [0 if l is None else int(l[1].shape[0]) for l in lists]
            order = [None if l is None else l[0] for l in lists]
            offsets = np.concatenate(([0], np.cumsum(counts))).astype(np.int32)
            if offsets[-1] > 0:
                slots = torch.cat([l[1] for l in lists if l is not None and l[1].shape[0] > 0]).to(torch.int32)
                type_offsets = torch.from_numpy(offsets).to(slots.device)
        if offsets[-1] > 0:
            # the tiled product for both: a row's result then does not depend on how many rows the batch has
            x_all = ops.project_typed_rows(flat_rep, slots, type_offsets, self.reductors, 1)
            g_all = None
            if with_forces:
                g_all = ops.project_typed_rows(rep_derivative.view(B * n * n * 3, -1), slots, type_offsets,
                                               self.reductors, 3 * n)
            mol_of_atom = torch.div(slots, n, rounding_mode='floor')
            for t in range(ne):
                if counts[t] == 0:
                    continue
                o0, o1 = int(offsets[t]), int(offsets[t + 1])
                sub_grad = g_all[o0 * 3 * n:o1 * 3 * n].view(o1 - o0, n, 3, -1) if with_forces else None
                items.append((order[t], mol_of_atom[o0:o1], x_all[o0:o1], sub_grad))
        return {'B': B, 'n': n, 'device': coordinates.device, 'items': items}

    def _rows_from_projected(self, proj, with_forces, zero_energy_rows=False):
        """fp64 row matrix [B (+ B*n*3), F] from the projected rows of one batch, at the current
        sigma: B energy rows, then the B*n*3 force rows in (molecule, atom, xyz) order
        (kernel.py:134-170)."""
        B, n, F = proj['B'], proj['n'], self.nfeatures()
        nrows = B + (B * n * 3 if with_forces else 0)
        own_force_rows = with_forces and self.writes_force_rows()
        if own_force_rows:
            rows = torch.empty(nrows, F, device=proj['device'], dtype=torch.float64)
            rows[:B].zero_()
        else:
            rows = torch.zeros(nrows, F, device=proj['device'], dtype=torch.float64)
        Zenergy = rows[:B]
        G = rows[B:].view(B, n, 3, F) if with_forces else None
        self._queue_force_rows = own_force_rows     # calculate_features may queue; finish_features runs the queue
        for e, batch_indexes, sub, sub_grad in proj['items']:
            self.calculate_features(sub, e, batch_indexes, Zenergy, sub_grad if with_forces else None, G)
        self._queue_force_rows = False
        self.finish_features(G, overwrite=own_force_rows)
        if zero_energy_rows:
            Zenergy.fill_(0)        # energy rows stay, as zeros, so the row count is unchanged (kernel.py:164-165)
        return rows

    def _batch_rows(self, data, with_forces, zero_energy_rows=False):
        """Rows of one formatted batch: representation (+ Jacobian), projection, features."""
        return self._rows_from_projected(self._batch_projected(data, with_forces), with_forces, zero_energy_rows)

    def _sort_species_tensor(self):
        """The model's elements as the float tensor `ops.element_types` compares charges with, in
        the order of the projection matrices (element2index)."""
        t = getattr(self, '_sort_species_cache', None)
        if t is None or t.device != self.reductors.device:
            vals = np.zeros(self.reductors.shape[0], dtype=np.float32)
            for e in self.elements:
                vals[int(self.element2index[int(e)])] = float(e)
            t = torch.from_numpy(vals).to(self.reductors.device)
            self._sort_species_cache = t
        return t

    @staticmethod
    def _element_index(data, charges, e):
        """Flat (molecule-major) indices of the atoms of element e by a device search (the reductor
        fit, and batches that did not come from `format_data`)."""
        return torch.nonzero(charges.reshape(-1).int() == e).reshape(-1)

    # -- training -------------------------------------------------------------------------
    def build_Z_components(self, X, Q, E=None, F=None, cells=None, inv_cells=None, print_info=True, cpu_solve=False,
                           ntiles=1, use_specialized_matmul=False):
        """Z^T Z [F,F] and Z^T y [F,1] in fp64 over the training set (kernel.py:46-217).

        X, Q: lists of [natoms_i,3] coordinates / [natoms_i] charges; E, F: energies /
        forces (either may be None).  cpu_solve keeps Z^T Z on the host; ntiles > 1 builds
        it in row blocks of ceil(nfeatures/ntiles) features; use_specialized_matmul takes
        the fp32-Kahan -> fp64 product instead of the fp64 one.
        """
        if self.reductors is None:
            raise RuntimeError("ERROR: Must call model.get_reductors() first to initialize the projection matrices.")
        if E is None and F is None:
            raise RuntimeError("ERROR: must have either E, F or both as input to train().")
        nf = self.nfeatures()
        dev = self.device
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        ZTZ = torch.zeros(nf, nf, device=torch.device('cpu') if cpu_solve else dev, dtype=torch.float64)
        ZtrainY = torch.zeros(nf, 1, device=dev, dtype=torch.float64)
        start.record()
        mirror_pending = False
        nsub = int(np.ceil(nf / ntiles))
        for tile in range(ntiles):
            lo, hi = tile * nsub, min(nsub * (tile + 1), nf)
            if ntiles > 1:
                if print_info:
                    print("tile:", tile + 1, "of", ntiles, "tiles, tile size:", hi - lo)
                ZTZ_tile = torch.zeros(hi - lo, nf, device=dev, dtype=torch.float64)
            for i in self._progress(range(0, len(X), self.nbatch_train), print_info):
                sl = slice(i, i + self.nbatch_train)
                data = self.format_data(X[sl], Q[sl], E=E[sl] if E is not None else None,
                                        F=F[sl] if F is not None else None,
                                        cells=cells[sl] if cells is not None else None,
                                        inv_cells=inv_cells[sl] if cells is not None else None)
                zbatch = data['charges'].shape[0]
                targets = self._targets(data, zbatch, E is not None, F is not None)
                rows = self._batch_rows(data, F is not None, zero_energy_rows=E is None)
                if ntiles > 1:
                    if use_specialized_matmul:
                        matmul_and_reduce(rows[:, lo:hi].float().T.contiguous(), rows.float(), ZTZ_tile)
                        ZtrainY[lo:hi] += torch.matmul(rows[:, lo:hi].T, targets)
                    else:
                        ops.gram(rows, targets, ZTZ_tile, ZtrainY, f0=lo, f1=hi)
                elif cpu_solve:
                    part = torch.zeros(nf, nf, device=dev, dtype=torch.float64)
                    ops.gram(rows, targets, part, ZtrainY)
                    ZTZ += part.cpu()
                elif use_specialized_matmul:
                    r32 = rows.float()
                    matmul_and_reduce(r32.T.contiguous(), r32, ZTZ)
                    ZtrainY += torch.matmul(rows.T, targets)
                else:
                    ops.gram(rows, targets, ZTZ, ZtrainY, mirror=False)    # upper tiles; mirrored once below
                    mirror_pending = True
                del rows
            if ntiles > 1:
                ZTZ[lo:hi, :] += ZTZ_tile.cpu() if cpu_solve else ZTZ_tile
        if mirror_pending:
            ops.gram_mirror(ZTZ)
        end.record()
        torch.cuda.synchronize()
        if print_info:
            print("ZTZ time: ", start.elapsed_time(end), "ms")
        return ZTZ, ZtrainY

    @staticmethod
    def _progress(it, show):
        if show:
            from tqdm import tqdm
            return tqdm(it)
        return it

    def _targets(self, data, zbatch, has_E, has_F):
        """Target column in the row order of `_batch_rows` (kernel.py:118-124)."""
        energies, forces = data['energies'], data['forces']
        if has_E and not has_F:
            return energies[:, None]
        if has_F and not has_E:
            zero = torch.zeros((zbatch, 1), device=forces.device, dtype=torch.float64)
            return torch.cat((zero, forces.flatten()[:, None]), dim=0)
        return torch.cat((energies[:, None], forces.flatten()[:, None]), dim=0)

    def train(self, X, Q, E=None, F=None, cells=None, inv_cells=None, print_info=True, cpu_solve=False, ntiles=1,
              use_specialized_matmul=False):
        """alpha = (Z^T Z + lambda I)^-1 Z^T y (kernel.py:219-247)."""
        ZTZ, ZtrainY = self.build_Z_components(X, Q, E, F, cells, inv_cells, print_info, cpu_solve, ntiles,
                                               use_specialized_matmul=use_specialized_matmul)
        ZTZ.diagonal().add_(self.llambda)
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        start.record()
        if cpu_solve:
            self.alpha = torch.linalg.solve(ZTZ, ZtrainY.cpu())[:, 0].to(self.device)
        else:
            self.alpha = self._solve_spd(ZTZ, ZtrainY, overwrite_a=True)[:, 0]     # Z^T Z is not needed again
        end.record()
        torch.cuda.synchronize()
        if print_info:
            print("coefficients time: ", start.elapsed_time(end), "ms")
        self.is_trained = True

    @staticmethod
    def _solve_spd(A, b, overwrite_a=False):
        """x = A^-1 b for the regularised normal matrix.  The reference calls
        torch.linalg.solve (LU, kernel.py:231); Z^T Z + lambda I is symmetric positive definite,
        so the library's blocked Cholesky factorisation gives the same solution for half the
        flops; LU remains the fallback when rounding has left the matrix numerically indefinite.

        overwrite_a: A (symmetric, both triangles stored) may be used up.  The factorisation then
        works in A itself instead of in a copy of it (2 GB at 16 384 features); it touches the
        upper triangle and the 128 x 128 tiles on the diagonal only, so those tiles are kept aside
        (16 MB) and, should a pivot fail, A is put together again from them and its lower
        triangle before LU takes it."""
        if A.is_cuda and b.dim() == 2 and b.shape[1] == 1 and A.stride(1) == 1 and A.stride(0) % 2 == 0:
            if not overwrite_a:
                x, info = ops.cholesky_solve_spd(A, b)
                if int(info.item()) == 0:
                    return x
                return torch.linalg.solve(A, b)
            n, ld, t = int(A.shape[0]), int(A.stride(0)), 128
            whole = n // t
            tiles = A.as_strided((whole, t, t), (t * (ld + 1), ld, 1))
            kept = tiles.clone()
            last = A[whole * t:, whole * t:].clone()
            x, info = ops.cholesky_solve_spd(A, b, overwrite_a=True)
            if int(info.item()) == 0:
                return x
            low = torch.tril(A, -1)
            A.copy_(low + low.T)
            del low
            tiles.copy_(kept)
            A[whole * t:, whole * t:] = last
            return torch.linalg.solve(A, b)
        L, info = torch.linalg.cholesky_ex(A)
        if int(info.item()) == 0:
            return torch.cholesky_solve(b, L)
        return torch.linalg.solve(A, b)

    def hyperparam_opt_nested_cv(self, X, Q, E, F=None, cells=None, inv_cells=None,
                                 sigmas=np.linspace(1.5, 12.5, 10), lambdas=np.logspace(-11, -5, 9), kfolds=5,
                                 print_info=True, use_rmse=False):
        """K-fold grid search over (sigma, lambda) (kernel.py:249-347)."""
        from sklearn.model_selection import KFold
        kf = KFold(n_splits=kfolds, shuffle=False)
        best = (None, None, np.inf)
        pick = lambda seq, ids: [seq[z] for z in ids]
        err = torch.sqrt if use_rmse else (lambda v: v)
        red = (lambda d: torch.mean(d * d)) if use_rmse else (lambda d: torch.mean(torch.abs(d)))
        # sigma enters through the coefficient normalisation alone (hadamard_features.py:68,93), so
        # per fold the representation, its Jacobian and the projected rows are built ONCE and kept;
        # per sigma only the features and Z^T Z / Z^T y are redone, and those serve the whole lambda
        # row (the reference rebuilds everything for every grid point).  For the RFF model W is drawn
        # with the sigma of construction (random_features.py:54): assigning self.sigma here does not
        # change it, as in the reference; call sample_elemental_basis() per sigma for a real scan.
        nf = self.nfeatures()
        fold_errors = np.zeros((len(sigmas), len(lambdas)))
        for train_index, test_index in kf.split(X):
            Xtr, Qtr, Etr = pick(X, train_index), pick(Q, train_index), pick(E, train_index)
            Ftr = pick(F, train_index) if F is not None else None
            cached = self._projected_batches(Xtr, Qtr, Etr, Ftr, cells, inv_cells)
            Xt, Qt = pick(X, test_index), pick(Q, test_index)
            data = self.format_data(Xt, Qt, pick(E, test_index), pick(F, test_index) if F is not None else None,
                                    cells=cells, inv_cells=inv_cells)
            max_natoms = int(data['natom_counts'].max().item())
            for si, sigma in enumerate(sigmas):
                self.sigma = sigma
                if cached is None:          # the projected rows of this fold would not fit the cache budget
                    ZTZ, ZtrainY = self.build_Z_components(Xtr, Qtr, Etr, Ftr, cells, inv_cells, print_info=False)
                else:
                    ZTZ = torch.zeros(nf, nf, device=self.device, dtype=torch.float64)
                    ZtrainY = torch.zeros(nf, 1, device=self.device, dtype=torch.float64)
                    for proj, targets in cached:
                        rows = self._rows_from_projected(proj, F is not None)
                        ops.gram(rows, targets, ZTZ, ZtrainY, mirror=False)
                        del rows
                    ops.gram_mirror(ZTZ)
                diag = ZTZ.diagonal().clone()
                for li, llambda in enumerate(lambdas):
                    self.llambda = llambda
                    ZTZ.diagonal().copy_(diag + llambda)
                    self.alpha = self._solve_spd(ZTZ, ZtrainY)[:, 0]
                    self.is_trained = True
                    if F is not None:
                        ep, fp = self.predict(Xt, Qt, max_natoms, cells=cells, inv_cells=inv_cells, forces=True,
                                              print_info=False)
                        e_err = err(red(ep - data['energies']))
                        f_err = err(red(fp - data['forces']))
                        fold_errors[si, li] += 0.5 * float(e_err + f_err)
                    else:
                        ep = self.predict(Xt, Qt, max_natoms, cells=cells, inv_cells=inv_cells, forces=False,
                                          print_info=False)
                        fold_errors[si, li] += float(err(red(ep - data['energies'])))
                del ZTZ, ZtrainY
            del cached
        for si, sigma in enumerate(sigmas):
            for li, llambda in enumerate(lambdas):
                fold_error = fold_errors[si, li] / kfolds
                if print_info:
                    print("sigma", sigma, "lambda", llambda, "error", fold_error)
                if fold_error < best[2]:
                    best = (sigma, llambda, fold_error)
        if print_info:
            print("Best error: ", best[2], "sigma = ", best[0], "lambda = ", best[1])
        return best[0], best[1]

    #: upper bound, in bytes, on the projected rows (all training batches of one fold) the grid search keeps
    #: on the device; the budget actually used is the smaller of this and half of the device memory that
    #: is free once one batch's transient arrays (dense Jacobian, fp64 row matrix) are set aside
    grid_search_cache_bytes = 64 << 30

    def _grid_search_budget(self, nmax, with_forces):
        budget = int(self.grid_search_cache_bytes)
        if torch.cuda.is_available() and self.device.type == "cuda":
            free, _ = torch.cuda.mem_get_info(self.device)
            free += torch.cuda.memory_reserved(self.device) - torch.cuda.memory_allocated(self.device)
            nb = int(self.nbatch_train)
            rows = nb * (1 + (3 * nmax if with_forces else 0))
            transient = 8 * rows * self.nfeatures()                                     # fp64 row matrix of a batch
            if with_forces:
                transient += 4 * nb * nmax * nmax * 3 * self.rep.get_repsize()          # its dense Jacobian
            budget = min(budget, max(0, (free - transient) // 2))
        return budget

    def _projected_batches(self, X, Q, E, F, cells, inv_cells):
        """[(projected rows, targets)] of every training batch, or None (the caller then rebuilds
        the rows per grid point) when they would take more than the budget (per atom: npcas
        floats, times 1 + 3 n with forces) or the device runs out of memory while building them."""
        nmax = max((len(q) for q in Q), default=0)
        natoms = sum(len(q) for q in Q)
        need = 4 * self.npcas * natoms * (1 + (3 * nmax if F is not None else 0))
        if need > self._grid_search_budget(nmax, F is not None):
            return None
        out = []
        try:
            for i in range(0, len(X), self.nbatch_train):
                sl = slice(i, i + self.nbatch_train)
                data = self.format_data(X[sl], Q[sl], E=E[sl] if E is not None else None,
                                        F=F[sl] if F is not None else None,
                                        cells=cells[sl] if cells is not None else None,
                                        inv_cells=inv_cells[sl] if cells is not None else None)
                targets = self._targets(data, data['charges'].shape[0], E is not None, F is not None)
                out.append((self._batch_projected(data, F is not None), targets))
        except torch.cuda.OutOfMemoryError:
            del out
            torch.cuda.empty_cache()
            return None
        return out

    #: atoms the fused predict route aims to put into one launch chain (see _fused_batch)
    fused_batch_atoms = 131072

    def _fused_batch(self, max_natoms):
        """Molecules per batch of the list-route `predict` on the fused route: nbatch_test, raised
        to about `fused_batch_atoms` atoms.  nbatch_test bounds the reference's per-batch
        [atoms, features] arrays (64 by default, hadamard_features.py:17); the fused chain keeps
        none of them (some 6 KB per atom), and batches of 64 molecules leave the chip mostly idle."""
        return max(int(self.nbatch_test), self.fused_batch_atoms // max(int(max_natoms), 1))

    # -- explicit-Jacobian predict route ----------------------------------------------------
    def predict_cuda(self, X, Q, max_natoms, cells=None, inv_cells=None, forces=False, print_info=True):
        """fp64 energies [N] (and forces [N,max_natoms,3]) as Z.alpha and G.alpha
        (kernel.py:349-445)."""
        if self.is_trained is False:
            raise RuntimeError("Error: must train the model first by calling train()!")
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        predict_energies = torch.zeros(len(X), device=self.device, dtype=torch.float64)
        predict_forces = torch.zeros(len(X), max_natoms, 3, device=self.device, dtype=torch.float64)
        alpha = self.alpha.double()
        start.record()
        for i in self._progress(range(0, len(X), self.nbatch_test), print_info):
            sl = slice(i, i + self.nbatch_test)
            data = self.format_data(X[sl], Q[sl], cells=cells[sl] if cells is not None else None,
                                    inv_cells=inv_cells[sl] if cells is not None else None)
            B, n = data['charges'].shape
            rows = self._batch_rows(data, forces is True)
            out = torch.matmul(rows, alpha)
            predict_energies[sl] = out[:B]
            if forces is True:
                predict_forces[sl, :n] = out[B:].reshape(B, n, 3)
        end.record()
        torch.cuda.synchronize()
        if print_info:
            print("prediction for", len(X), "molecules time: ", start.elapsed_time(end), "ms")
        if forces is True:
            return (predict_energies, predict_forces)
        return predict_energies

    # -- reductors ----------------------------------------------------------------------
    def get_reductors(self, X, Q, cells=None, inv_cells=None, npcas=128, npca_choice=256, nsamples=4096,
                      print_info=True):
        """Per element: left singular vectors of a [repsize, nselected] sample of atomic
        representations, first `npcas` columns, no mean-centring (kernel.py:447-540)."""
        for e in self.elements:
            element_idx = self.element2index[int(e)]
            ids = np.array([i for i in range(len(Q)) if int(e) in Q[i]], dtype=np.int64)
            if len(ids) == 0:
                continue
            pick = np.random.choice(ids, size=min(len(ids), 1024))
            sub_X = [X[i] for i in pick]
            sub_Q = [Q[i] for i in pick]
            chunks, nselected = [], 0
            for i in range(0, len(sub_X), self.nbatch_train):
                if nselected > nsamples:
                    break
                data = self.format_data(sub_X[i:i + self.nbatch_train], sub_Q[i:i + self.nbatch_train], cells=cells,
                                        inv_cells=inv_cells)
                rep = self.rep.get_representation(data['coordinates'], data['charges'], data['atomIDs'],
                                                  data['molIDs'], data['natom_counts'], data['cells'],
                                                  data['inv_cells'])
                idx = self._element_index(data, data['charges'], int(e))
                if idx.shape[0] == 0:
                    continue
                rows = rep.view(-1, rep.shape[-1]).index_select(0, idx)
                rows = rows[torch.randperm(rows.shape[0], device=rows.device)[:npca_choice]]
                nselected += rows.shape[0]
                chunks.append(rows)
            if not chunks:
                continue
            mat = torch.cat(chunks)
            U, S = self._left_singular_vectors(mat)
            reductor = U[:, :npcas]
            if print_info:
                cev = 100 - (S.sum() - S[:npcas].sum()) / S.sum() * 100
                print(f"element {int(e)}: {reductor.shape[0]} -> {reductor.shape[1]}  "
                      f"Cumulative Explained Feature Variance = {float(cev):6.2f} %")
            if reductor.shape[1] < npcas:
                raise RuntimeError(f"ERROR - not enough atomic environments in input dataset for element {int(e)}. "
                                   "Either increase npca_choice or provide more structures.")
            self.reductors[element_idx] = reductor

    @staticmethod
    def _left_singular_vectors(mat):
        """Left singular vectors and singular values of mat.T for mat [nsamples, repsize], in
        descending order: what torch.linalg.svd(mat.T) returns in the reference (kernel.py:509).
        Computed as the eigenvectors of the repsize x repsize fp64 matrix mat^T mat (the library's
        Gram kernel, then a small symmetric eigensolve) instead of an SVD of the tall matrix.
        The sign of a singular vector is arbitrary in any SVD; here its largest component is
        made positive, so equal inputs give equal reductors."""
        rows = mat.double().contiguous()
        R = rows.shape[1]
        cov = torch.zeros(R, R, dtype=torch.float64, device=rows.device)
        ops.gram(rows, None, cov, None)
        w, V = torch.linalg.eigh(cov)
        w, V = w.flip(0), V.flip(1)
        lead = V.gather(0, V.abs().argmax(dim=0, keepdim=True))
        V = V * torch.where(lead < 0, -1.0, 1.0)
        k = min(rows.shape)                      # an SVD of [repsize, nsamples] has min(...) vectors
        return V[:, :k].to(mat.dtype), torch.sqrt(w[:k].clamp_min(0.0)).to(mat.dtype)

    # -- model files ------------------------------------------------------------------------
    def _fill_from_attribute_tree(self, tree, tensors):
        """Copy what a saved model carries beside its feature tensors (kernel.py:24-41 of the
        reference: reductors, element2index, self_energy, unit flags, alpha) and the feature
        tensors named in `tensors` ({attribute: dtype}), checking every shape against the one
        this model was constructed with."""
        dev = self.device
        for name, dtype in dict(tensors, reductors=torch.float32).items():
            have = getattr(self, name)
            new = torch.from_numpy(np.ascontiguousarray(tree[name])).to(dtype)
            if tuple(new.shape) != tuple(have.shape):
                raise ValueError("model file: %s has shape %s, the hyper-parameters give %s"
                                 % (name, tuple(new.shape), tuple(have.shape)))
            setattr(self, name, new.to(dev))
        e2i = torch.from_numpy(np.asarray(tree["element2index"], dtype=np.int64))
        if not torch.equal(e2i, self.element2index):
            raise ValueError("model file: element2index does not follow from its element list")
        alpha = torch.from_numpy(np.ascontiguousarray(tree["alpha"]))          # fp64 once trained
        if alpha.shape != (self.nfeatures(),):
            raise ValueError("model file: alpha has %d entries for %d features" % (alpha.numel(), self.nfeatures()))
        self.alpha = alpha.to(dev)
        self.is_trained = bool(tree.get("is_trained", True))
        se = tree.get("self_energy")
        self.self_energy = None if se is None else torch.from_numpy(np.asarray(se, dtype=np.float64))
        self._convert_from_hartree_to_kcal = bool(tree.get("_convert_from_hartree_to_kcal", False))
        self._subtract_self_energies = bool(tree.get("_subtract_self_energies", False))
        self.hartree2kcalmol = float(tree.get("hartree2kcalmol", 627.5))
        return self

    # -- unit conversion / self energies ----------------------------------------------------
    def set_subtract_self_energies(self, subtract):
        self._subtract_self_energies = subtract

    def subtract_self_energies(self):
        return self._subtract_self_energies

    def set_convert_hartree2kcal(self, convert):
        self._convert_from_hartree_to_kcal = convert

    def convert_hartree2kcal(self):
        return self._convert_from_hartree_to_kcal

    def calculate_self_energy(self, Q, E):
        """Least-squares per-element contribution to E (kernel.py:554-599)."""
        counts = torch.zeros(len(Q), len(self.elements), dtype=torch.float64)
        for i, q in enumerate(Q):
            q = np.asarray(q)
            for j, e in enumerate(self.elements):
                counts[i, j] = float((q == int(e)).sum())
        energies = torch.tensor(np.asarray(E, dtype=np.float64))
        if self.convert_hartree2kcal():
            energies = energies * self.hartree2kcalmol
        XTX = counts.T @ counts
        beta = torch.linalg.lstsq(XTX, counts.T @ energies[:, None]).solution[:, 0]
        species = self.elements.long()
        self.self_energy = torch.zeros(int(torch.max(species)) + 1, dtype=torch.float64)
        self.self_energy[species] = beta
        print("Self Energies: ", self.self_energy)

    # -- batch formatting -------------------------------------------------------------------
    def _format_padded_arrays(self, X, Q, E=None, F=None, cells=None, inv_cells=None):
        """format_data for a batch that already is one zero-padded array pair X [B,n,3], Q [B,n]
        (charge 0 = padding, real atoms first in every row: the layout format_data itself
        produces, kernel.py:630-695), with energies E [B] and forces F [B,n,3] (zero-padded) when
        it is a training batch.  One upload per array; counts, atom and molecule indices, the
        self-energy correction and the unit conversion are done on the device, with no Python loop
        over molecules; the per-element atom index is left to a device sort (`_batch_projected`),
        for which only the element counts are taken here, from the host copy of the charges."""
        dev = self.device
        B, n = Q.shape
        coords = torch.from_numpy(np.ascontiguousarray(X, dtype=np.float32)).to(dev)
        charges = torch.from_numpy(np.ascontiguousarray(Q, dtype=np.float32)).to(dev)
        mask = charges > 0
        counts = mask.sum(dim=1, dtype=torch.int32)
        hostmask = np.asarray(Q) > 0
        if hostmask.all():                                 # fixed composition: no search needed
            flat = torch.arange(B * n, device=dev)
        else:
            # padding must trail the real atoms of its row
            if (hostmask[:, 1:] & ~hostmask[:, :-1]).any():
                raise RuntimeError("format_data: padded rows must hold their real atoms first")
            flat = mask.reshape(-1).nonzero()[:, 0]
        data = {
            'coordinates': coords,
            'charges': charges,
            'natom_counts': counts,
            'atomIDs': (flat % n).to(torch.int32),
            'molIDs': (flat // n).to(torch.int32),
            'energies': None,
            'forces': None,
            'cells': torch.empty((0, 3, 3), device=dev),
            'inv_cells': torch.empty((0, 3, 3), device=dev),
        }
        if E is not None or F is not None:
            data['element_counts'] = self._element_counts(np.asarray(Q).reshape(-1))
        if E is not None:
            energies = torch.from_numpy(np.ascontiguousarray(E, dtype=np.float64).reshape(B)).to(dev)
            if self.convert_hartree2kcal():
                energies = energies * self.hartree2kcalmol
            if self.subtract_self_energies():
                se = self.self_energy.to(dev)
                energies = energies - se[charges.long()].sum(dim=1)        # se[0] = 0: padding adds nothing
            data['energies'] = energies
        if F is not None:
            Fa = np.asarray(F, dtype=np.float64)
            if Fa.shape != (B, n, 3):
                raise RuntimeError("format_data: forces of a padded batch must be one [B, n, 3] array, got %s"
                                   % (Fa.shape,))
            forces = torch.from_numpy(np.ascontiguousarray(Fa)).to(dev)
            if self.convert_hartree2kcal():
                forces = forces * self.hartree2kcalmol
            data['forces'] = forces * mask[:, :, None]                      # padded slots carry no target
        if cells is not None:
            data['cells'] = torch.from_numpy(np.asarray(cells, dtype=np.float32).reshape(B, 3, 3)).to(dev)
            data['inv_cells'] = torch.from_numpy(np.asarray(inv_cells, dtype=np.float32).reshape(B, 3, 3)).to(dev)
        return data

    def _element_counts(self, flat_charges):
        """{element: number of atoms} of a batch from the host copy of its charges (one bincount)."""
        q = np.asarray(flat_charges).astype(np.int64, copy=False)
        hist = np.bincount(q[q >= 0], minlength=int(self.element2index.shape[0]))
        return {int(e): int(hist[int(e)]) for e in self.elements}

    @staticmethod
    def _concat_rows(items, width, dtype):
        """All per-molecule arrays stacked into one [total_atoms, width] array.  One
        np.concatenate over the sequence (a C loop) when the items already have the expected
        shape; a per-item conversion only for odd inputs (nested lists, flattened rows)."""
        try:
            out = np.concatenate(items)
            if out.ndim == (2 if width > 1 else 1) and (width == 1 or out.shape[1] == width):
                return out.astype(dtype, copy=False).reshape(-1, width)
        except ValueError:
            pass
        return np.concatenate([np.asarray(v, dtype=dtype).reshape(-1, width) for v in items])

    def format_data(self, X, Q, E=None, F=None, cells=None, inv_cells=None):
        """Lists of per-molecule arrays -> zero-padded device tensors with the keys
        coordinates / charges / natom_counts / atomIDs / molIDs / energies / forces /
        cells / inv_cells (kernel.py:601-722), plus, for a training batch, 'element_counts':
        {element: number of its atoms}, so that the element-sorted atom index can be built by a
        device sort without a host round trip.  X [B,n,3] and Q [B,n] given as zero-padded
        arrays (with E [B], F [B,n,3]) are uploaded as they are."""
        if self.subtract_self_energies() and self.self_energy is None:
            raise RuntimeError("ERROR: must call model.calculate_self_energy first - this computes atomic "
                               "contributes to the potential energy.")
        dev = self.device
        zbatch = len(X)
        if isinstance(X, np.ndarray) and X.ndim == 3 and isinstance(Q, np.ndarray) and Q.ndim == 2:
            return self._format_padded_arrays(X, Q, E, F, cells, inv_cells)
        counts = np.fromiter(map(len, X), dtype=np.int32, count=zbatch)
        n = int(counts.max()) if zbatch else 0
        if zbatch and n > 0 and int(counts.min()) == n:
            # molecules of one size (a trajectory, a fixed composition): the lists stacked are the padded
            # array pair already, with nothing to pad and no index to build on the host
            try:
                Xa = self._concat_rows(X, 3, np.float32).reshape(zbatch, n, 3)
                Qa = self._concat_rows(Q, 1, np.float32).reshape(zbatch, n)
                Fa = None if F is None else self._concat_rows(F, 3, np.float64).reshape(zbatch, n, 3)
                Ea = None if E is None else np.asarray(E, dtype=np.float64).reshape(zbatch)
                if (Qa > 0).all():
                    return self._format_padded_arrays(Xa, Qa, Ea, Fa, cells, inv_cells)
            except ValueError:
                pass                                        # odd shapes: the general route sorts them out or raises
        # one concatenation and one scatter instead of a Python loop over molecules
        molIDs = np.repeat(np.arange(zbatch, dtype=np.int32), counts)
        starts = np.cumsum(counts) - counts
        atomIDs = (np.arange(int(counts.sum()), dtype=np.int64) - np.repeat(starts, counts)).astype(np.int32)
        flat = molIDs.astype(np.int64) * n + atomIDs
        coords = np.zeros((zbatch, n, 3), dtype=np.float32)
        charges = np.zeros((zbatch, n), dtype=np.float32)
        if zbatch:
            coords.reshape(-1, 3)[flat] = self._concat_rows(X, 3, np.float32)
            charges.reshape(-1)[flat] = self._concat_rows(Q, 1, np.float32).reshape(-1)
        data = {
            'coordinates': torch.from_numpy(coords).to(dev),
            'charges': torch.from_numpy(charges).to(dev),
            'natom_counts': torch.from_numpy(counts).to(dev),
            'atomIDs': torch.from_numpy(atomIDs).to(dev),
            'molIDs': torch.from_numpy(molIDs).to(dev),
            'energies': None,
            'forces': None,
            'cells': torch.empty((0, 3, 3), device=dev),
            'inv_cells': torch.empty((0, 3, 3), device=dev),
        }
        flat_q = charges.reshape(-1).astype(np.int64)
        if E is not None or F is not None:
            # training batches gather rows per element: the element-sorted atom index is built on the
            # device (`_batch_projected`), which needs only the per-element counts from here
            data['element_counts'] = self._element_counts(flat_q)
        if E is not None:
            energies = np.array(E, dtype=np.float64).reshape(zbatch).copy()
            if self.convert_hartree2kcal():
                energies *= self.hartree2kcalmol
            if self.subtract_self_energies():
                se = self.self_energy.numpy()
                energies -= np.bincount(molIDs, weights=se[flat_q[flat]], minlength=zbatch)
            data['energies'] = torch.from_numpy(energies).to(dev)
        if F is not None:
            forces = np.zeros((zbatch, n, 3), dtype=np.float64)
            if zbatch:
                forces.reshape(-1, 3)[flat] = self._concat_rows(F, 3, np.float64)
            if self.convert_hartree2kcal():
                forces *= self.hartree2kcalmol
            data['forces'] = torch.from_numpy(forces).to(dev)
        if cells is not None:
            data['cells'] = torch.from_numpy(np.asarray(cells, dtype=np.float32).reshape(zbatch, 3, 3)).to(dev)
            data['inv_cells'] = torch.from_numpy(np.asarray(inv_cells, dtype=np.float32).reshape(zbatch, 3, 3)).to(dev)
        return data
