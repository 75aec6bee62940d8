"""RandomFourrierFeaturesModel (qml_lightning/models/random_features.py:17-236): features
sqrt(2/F) cos(x W + b) with W ~ N(0,1)/(2 sigma^2) per element."""
from typing import Final, Optional

import numpy as np
import torch

from .. import ops
from ..cuda.rff_gpu import get_rff
from ..representations.dimensionality_reduction import project_representation
from . import hadamard_features  # noqa: F401  (registers the fused operators)
from .hadamard_features import _no_cells
from .kernel import BaseKernel, _default_device, alpha_f32, rep_from_attribute_tree


class RandomFourrierFeaturesModel(BaseKernel, torch.nn.Module):
    """`fused=True` runs forward() through one matrix-core kernel that never writes the
    [atoms, nfeatures] matrix; it exists for npcas 64 or 128 and a multiple of 32 features and
    raises for other shapes.  `fused=False` is the reference's own operator sequence (library
    GEMM).  `fused=None` (default) takes the fused kernel where it exists."""

    fused: Final[bool]
    separate_ops: Final[bool]

    def __init__(self, rep=None, elements=np.array([1, 6, 7, 8]), sigma=2.0, llambda=1e-10,
                 nstacks=8192, npcas=128, nbatch_train=64, nbatch_test=64, fused=None,
                 separate_ops=False):
        torch.nn.Module.__init__(self)
        BaseKernel.__init__(self, rep, npcas, elements, sigma, llambda)
        self.device = _default_device()
        self.npcas = npcas
        has_kernel = npcas in (64, 128) and (nstacks * npcas) % 32 == 0
        if fused and not has_kernel:
            raise ValueError("RandomFourrierFeaturesModel(fused=True): the fused kernel exists for npcas 64 or 128 and a "
                             "multiple of 32 features, not npcas = %d with %d features; pass fused=False for the "
                             "operator sequence of the reference" % (npcas, nstacks * npcas))
        self.fused = has_kernel if fused is None else bool(fused)
        self.separate_ops = separate_ops   # fused route as five operators (one node each) instead of one
        self.nbatch_train = nbatch_train
        self.nbatch_test = nbatch_test
        self._nfeatures = nstacks * self.npcas
        self.species = torch.from_numpy(np.asarray(elements)).float().to(self.device)
        self.sort_species = hadamard_features.model_species_for_sort(self.species, rep)
        self.sample_elemental_basis()
        self.feature_normalisation = float(np.sqrt(2.0 / self._nfeatures))
        self.is_trained = False
        self.alpha = torch.zeros(self._nfeatures, device=self.device, dtype=torch.float)

    @torch.jit.unused
    def sample_elemental_basis(self):
        """W [ne,d,F] = N(0,1)/(2 sigma^2), b [ne,F] = U(0,2pi) (random_features.py:42-55)."""
        D, d = self.nfeatures(), self.npcas
        self.W = torch.zeros((len(self.elements), d, D), dtype=torch.float32, device=self.device)
        self.b = torch.zeros((len(self.elements), D), dtype=torch.float32, device=self.device)
        for e in self.elements:
            idx = self.element2index[int(e)]
            self.W[idx] = torch.from_numpy(np.random.normal(0.0, 1.0, [d, D]) / (2 * self.sigma ** 2)).to(self.device)
            self.b[idx] = torch.from_numpy(np.random.uniform(0.0, 1.0, [D]) * 2.0 * np.pi).to(self.device)

    def nfeatures(self):
        return self._nfeatures

    @torch.jit.unused
    def calculate_features(self, rep, element, indexes, feature_matrix, grad=None, derivative_matrix=None):
        """fp64 features / force features of one element (random_features.py:60-67)."""
        idx = self.element2index[int(element)]
        W, b = self.W[idx].double(), self.b[idx].double()
        get_rff(rep, W, b, indexes, feature_matrix)
        if derivative_matrix is not None and grad is not None:
            # the batch's atoms are molecule-major: atomic-free matrix-core kernel
            ops.rff_derivative_features(rep, grad, W, b, indexes, derivative_matrix, molecule_major=True)

    def forward(self, X, Z, atomIDs, molIDs, atom_counts, cell: Optional[torch.Tensor] = None,
                inv_cell: Optional[torch.Tensor] = None):
        """Total energies [B], differentiable in X; the feature GEMM is the BLAS library's
        (random_features.py:69-102)."""
        if cell is None:
            cell = torch.empty(0, 3, 3, device=X.device)
        if inv_cell is None:
            inv_cell = torch.empty(0, 3, 3, device=X.device)
        assert X.is_cuda, "X tensor must reside on GPU"
        assert Z.is_cuda, "Z tensor must reside on GPU"
        if self.fused and not self.separate_ops:
            # the whole chain below as ONE operator and one autograd node
            energies, _ = torch.ops.qml_lightning_sorf.fchl_rff_energy(
                X, Z, self.rep.species, atomIDs, molIDs, atom_counts, cell, inv_cell, self.rep.Rs2, self.rep.Rs3,
                self.rep.eta2, self.rep.eta3, self.rep.two_body_decay, self.rep.three_body_weight,
                self.rep.three_body_decay, self.rep.rcut, self.reductors, self.W, self.b, self.alpha.float(),
                self.sort_species, X.requires_grad)
            return energies
        torch_rep = self.rep.forward(X, Z, atomIDs, molIDs, atom_counts, cell, inv_cell)
        if self.fused:
            # atoms sorted by element on the device, projected with their own reductor into
            # compact rows, then one kernel for x.W + b -> cos -> alpha contraction (+ gradient)
            nslots = X.shape[0] * X.shape[1]
            flat_rep = torch_rep.view(nslots, torch_rep.shape[2])
            types = torch.ops.qml_lightning_fchl.get_element_types(X, Z, atom_counts, self.species).view(-1)
            slots = molIDs * X.shape[1] + atomIDs
            sorted_slots, type_offsets = torch.ops.qml_lightning_sorf.sort_by_type(types, slots,
                                                                                   self.reductors.shape[0])
            x = torch.ops.qml_lightning_sorf.project_typed(flat_rep, sorted_slots, type_offsets, self.reductors, types)
            e_slots, _ = torch.ops.qml_lightning_sorf.rff_energy_sorted(x, type_offsets, sorted_slots, self.W, self.b,
                                                                        self.alpha.float(), nslots, x.requires_grad)
            return e_slots.view(X.shape[0], X.shape[1]).sum(dim=1)
        # the reference's sequence (random_features.py:86-102); each element's atoms are looked up
        # once and gathered with index_select (backward: index_add, no second search)
        nmol, natoms_max = torch_rep.shape[0], torch_rep.shape[1]      # [1, n] for one unbatched molecule
        Ztest = torch.zeros(nmol, self.nfeatures(), device=X.device, dtype=torch.float32)
        flat_rep = torch_rep.view(nmol * natoms_max, torch_rep.shape[2])
        flat_charges = Z.int().view(-1)
        for e in self.elements:
            element_idx = self.element2index[e]
            atom_rows = torch.nonzero(flat_charges == e.item())[:, 0]
            if atom_rows.shape[0] == 0:
                continue
            batch_indexes = torch.div(atom_rows, natoms_max, rounding_mode='floor')
            sub = flat_rep.index_select(0, atom_rows)
            sub = project_representation(sub, self.reductors[element_idx])
            feats = self.feature_normalisation * torch.cos(torch.matmul(sub, self.W[element_idx])
                                                           + self.b[element_idx][None, :])
            Ztest = Ztest.index_add(0, batch_indexes, feats)
        return torch.matmul(Ztest, self.alpha.float())

    @torch.jit.unused
    def energies_and_forces(self, coordinates, charges, atomIDs, molIDs, natom_counts, cells=None, inv_cells=None,
                            forces=True):
        """(energies [B], forces [B,n,3] or None) for device tensors through the fused route,
        asynchronously on the current stream; no autograd graph (the fused kernel returns
        dE/dx itself)."""
        if cells is None or inv_cells is None:
            cells = inv_cells = _no_cells(coordinates.device)
        rep = self.rep
        with torch.no_grad():
            if forces:      # energies and -dE/dX from one operator, the sign applied in its last kernel
                return torch.ops.qml_lightning_sorf.fchl_rff_forces(
                    coordinates, charges, rep.species, atomIDs, molIDs, natom_counts, cells, inv_cells, rep.Rs2, rep.Rs3,
                    rep.eta2, rep.eta3, rep.two_body_decay, rep.three_body_weight, rep.three_body_decay, rep.rcut,
                    self.reductors, self.W, self.b, alpha_f32(self), self.sort_species)
            energies, _ = torch.ops.qml_lightning_sorf.fchl_rff_energy(
                coordinates, charges, rep.species, atomIDs, molIDs, natom_counts, cells, inv_cells, rep.Rs2, rep.Rs3,
                rep.eta2, rep.eta3, rep.two_body_decay, rep.three_body_weight, rep.three_body_decay, rep.rcut,
                self.reductors, self.W, self.b, alpha_f32(self), self.sort_species, False)
        return energies, None

    @torch.jit.unused
    def predict_opt(self, coordinates, charges, atomIDs, molIDs, natom_counts, zcells=None, zinv_cells=None,
                    forces=True, print_info=False, profiler=False):
        if self.is_trained is False:
            raise RuntimeError("Error: must train the model first by calling train()!")
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        start.record()
        if self.fused:
            result = self.energies_and_forces(coordinates, charges, atomIDs, molIDs, natom_counts, zcells, zinv_cells,
                                              forces=forces)
            end.record()
            torch.cuda.synchronize()
            if print_info:
                print("prediction for", coordinates.shape[0], "molecules time: ", start.elapsed_time(end), "ms")
            return result if forces else result[0]
        if forces:
            coordinates.requires_grad = True
        total_energies = self.forward(coordinates, charges, atomIDs, molIDs, natom_counts, zcells, zinv_cells)
        if forces:
            forces_torch, = torch.autograd.grad(-total_energies.sum(), coordinates)
        end.record()
        torch.cuda.synchronize()
        if print_info:
            print("prediction for", coordinates.shape[0], "molecules time: ", start.elapsed_time(end), "ms")
        return (total_energies, forces_torch) if forces else total_energies

    @torch.jit.unused
    def predict(self, X, Z, max_natoms, cells=None, inv_cells=None, forces=True, print_info=False):
        predict_energies = torch.zeros(len(X), device=self.device, dtype=torch.float32)
        predict_forces = torch.zeros(len(X), max_natoms, 3, device=self.device, dtype=torch.float32)
        step = self._fused_batch(max_natoms) if self.fused else self.nbatch_test
        for i in self._progress(range(0, len(X), step), print_info):
            sl = slice(i, i + step)
            data = self.format_data(X[sl], Z[sl], cells=cells[sl] if cells is not None else None,
                                    inv_cells=inv_cells[sl] if cells is not None else None)
            if self.fused:
                # no synchronisation per batch: the host formats the next batch while this one runs
                if self.is_trained is False:
                    raise RuntimeError("Error: must train the model first by calling train()!")
                result = self.energies_and_forces(data['coordinates'], data['charges'], data['atomIDs'],
                                                  data['molIDs'], data['natom_counts'], data['cells'],
                                                  data['inv_cells'], forces=forces)
                result = result if forces else result[0]
            else:
                result = self.predict_opt(data['coordinates'], data['charges'], data['atomIDs'], data['molIDs'],
                                          data['natom_counts'], data['cells'], data['inv_cells'], forces=forces)
            if forces:
                predict_energies[sl] = result[0].detach()
                predict_forces[sl, :result[1].shape[1]] = result[1]
            else:
                predict_energies[sl] = result.detach()
        torch.cuda.synchronize()
        if forces:
            return (predict_energies, predict_forces)
        return predict_energies

    @classmethod
    def from_reference_file(cls, file_name, fused=None, separate_ops=False):
        """A RandomFourrierFeaturesModel holding the weights of a model file written by
        `save_jit_model` (random_features.py:233-235 of the reference), read as data: see
        HadamardFeaturesModel.from_reference_file.  `nstacks` is recovered from the number of
        features the file's W has."""
        from ..utils import model_files
        tree = model_files.read_attribute_tree(file_name)
        if not str(tree.get("__class__", "")).endswith("RandomFourrierFeaturesModel"):
            raise ValueError("%s holds a %r, not a RandomFourrierFeaturesModel" % (file_name, tree.get("__class__")))
        rep = rep_from_attribute_tree(tree["rep"])
        npcas = int(tree["npcas"])
        nfeatures = int(np.asarray(tree["W"]).shape[2])
        if nfeatures % npcas != 0:
            raise ValueError("%s: %d features are not a multiple of npcas = %d" % (file_name, nfeatures, npcas))
        state = np.random.get_state()        # the constructor draws a W that is replaced at once
        try:
            model = cls(rep=rep, elements=np.asarray(tree["elements"], dtype=np.int64), sigma=float(tree["sigma"]),
                        llambda=float(tree["llambda"]), nstacks=nfeatures // npcas, npcas=npcas,
                        nbatch_train=int(tree["nbatch_train"]), nbatch_test=int(tree["nbatch_test"]), fused=fused,
                        separate_ops=separate_ops)
        finally:
            np.random.set_state(state)
        model._fill_from_attribute_tree(tree, {"W": torch.float32, "b": torch.float32})
        return model

    @torch.jit.unused
    def save_jit_model(self, file_name='model_rff.pt'):
        script = torch.jit.script(self)
        script.save(file_name)
