"""FCHLCuda: the reference's FCHL19 wrapper class (qml_lightning/representations/FCHL.py:16-133)
over the HIP kernels.  Same constructor arguments, attribute names/dtypes (they are what
`torch.jit.script` serialises) and method signatures."""
from typing import Optional

import numpy as np
import torch

from ..cuda import fchl_gpu, pairlist_gpu


def _default_device():
    return torch.device("cuda" if torch.cuda.is_available() else "cpu")


class FCHLCuda(torch.nn.Module):

    def __init__(self, species=np.array([1, 6, 7, 8]), rcut=6.0, nRs2=24, nRs3=20,
                 eta2=0.32, eta3=2.7, two_body_decay=1.8, three_body_weight=13.4, three_body_decay=0.57):
        super(FCHLCuda, self).__init__()
        dev = _default_device()
        self.species = torch.from_numpy(np.asarray(species)).float().to(dev)
        self.nspecies = len(species)
        # scalar hyper-parameters stay 0-d CPU tensors, as in the reference (FCHL.py:25-37)
        self.rcut = torch.tensor(rcut)
        self.nRs2 = torch.tensor(nRs2)
        self.nRs3 = torch.tensor(nRs3)
        self.eta2 = torch.tensor(eta2)
        self.eta3 = torch.tensor(eta3)
        self.two_body_decay = torch.tensor(two_body_decay)
        # the kernels take the weight with sqrt(eta3/pi) folded in (FCHL.py:35)
        self.three_body_weight = np.sqrt(eta3 / np.pi) * torch.tensor(three_body_weight)
        self.three_body_decay = torch.tensor(three_body_decay)
        self.Rs2 = torch.linspace(0.0, rcut, nRs2 + 1)[1:].to(dev)
        self.Rs3 = torch.linspace(0.0, rcut, nRs3 + 1)[1:].to(dev)
        self.fp_size = self.nspecies * nRs2 + (self.nspecies * (self.nspecies + 1)) * nRs3
        self.pi = (torch.acos(torch.zeros(1)) * 2).to(dev)
        self.device = dev

    def get_repsize(self):
        return self.fp_size

    @torch.jit.unused
    def get_neighbourlist(self, X, Z, max_neighbours, atom_counts, cell=None, inv_cell=None):
        return pairlist_gpu.get_neighbour_list_gpu(X, atom_counts, max_neighbours, self.rcut.item(), cell, inv_cell)

    @torch.jit.unused
    def get_neighbours(self, X, Z, atom_counts, cell=None, inv_cell=None):
        return pairlist_gpu.get_num_neighbours_gpu(X, atom_counts, self.rcut.item(), cell, inv_cell)

    @torch.jit.unused
    def get_element_types(self, X, Z, atom_counts):
        return fchl_gpu.get_element_types_gpu(X, Z, atom_counts, self.species)

    def _lists(self, X, Z, atom_counts, cell, inv_cell, nneighbours, neighbourlist):
        if nneighbours is None and neighbourlist is None:
            nneighbours = self.get_neighbours(X, Z, atom_counts, cell, inv_cell)
            max_neighbours = nneighbours.max().item()
            neighbourlist = self.get_neighbourlist(X, Z, max_neighbours, atom_counts, cell, inv_cell)
        return nneighbours, neighbourlist

    @torch.jit.unused
    def get_representation(self, X, Z, atomIDs, molIDs, atom_counts, cell=None, inv_cell=None, nneighbours=None,
                           neighbourlist=None):
        """rep f32 [B,n,R] (FCHL.py:66-80).  With no list given the kernel builds the
        neighbour lists itself; a given list is used as is."""
        element_types = self.get_element_types(X, Z, atom_counts)
        from .. import ops
        prm = ops.make_params(self.nspecies, self.Rs2, self.Rs3, self.eta2, self.eta3, self.two_body_decay,
                              self.three_body_weight, self.three_body_decay, self.rcut)
        return ops.fchl_forward(X, element_types, cell, inv_cell, atomIDs, molIDs, atom_counts, self.Rs2, self.Rs3,
                                prm, neighbourlist, nneighbours)

    @torch.jit.unused
    def get_representation_and_derivative(self, X, Z, atomIDs, molIDs, atom_counts, cell=None, inv_cell=None,
                                          nneighbours=None, neighbourlist=None):
        """(rep [B,n,R], grad [B,n,n,3,R]) (FCHL.py:82-97)."""
        element_types = self.get_element_types(X, Z, atom_counts)
        from .. import ops
        prm = ops.make_params(self.nspecies, self.Rs2, self.Rs3, self.eta2, self.eta3, self.two_body_decay,
                              self.three_body_weight, self.three_body_decay, self.rcut)
        rep, jac = ops.fchl_jacobian(X, element_types, cell, inv_cell, atomIDs, molIDs, atom_counts, self.Rs2,
                                     self.Rs3, prm, neighbourlist, nneighbours)
        return rep, jac

    @torch.jit.unused
    def rep_deriv_fd(self, X, Z, atomIDs, molIDs, natom_counts, cells=None, inv_cells=None, dx=0.005):
        """Central finite differences with the neighbour list frozen (FCHL.py:99-125)."""
        rep_derivative_fd = torch.zeros(X.shape[0], X.shape[1], X.shape[1], 3, self.fp_size, dtype=torch.float64,
                                        device=X.device)
        nneighbours, neighbourlist = self._lists(X, Z, natom_counts, cells, inv_cells, None, None)
        for i in range(X.shape[1]):
            for x in range(3):
                X_copy = X.clone()
                X_copy[:, i, x] += dx
                rep_plus = self.get_representation(X_copy, Z, atomIDs, molIDs, natom_counts, cells, inv_cells,
                                                   nneighbours, neighbourlist)
                X_copy[:, i, x] -= 2.0 * dx
                rep_minus = self.get_representation(X_copy, Z, atomIDs, molIDs, natom_counts, cells, inv_cells,
                                                    nneighbours, neighbourlist)
                rep_derivative_fd[:, :, i, x, :] = (rep_plus - rep_minus) / (2.0 * dx)
        return rep_derivative_fd

    def forward(self, X, Z, atomIDs, molIDs, atom_counts, cell: Optional[torch.Tensor] = None,
                inv_cell: Optional[torch.Tensor] = None):
        """Differentiable representation through the registered operator (FCHL.py:127-132)."""
        if cell is None:
            cell = torch.empty(0, 3, 3, device=X.device)
        if inv_cell is None:
            inv_cell = torch.empty(0, 3, 3, device=X.device)
        return torch.ops.qml_lightning_fchl.fchl_forwards(X, Z, self.species, atomIDs, molIDs, atom_counts, cell,
                                                          inv_cell, self.Rs2, self.Rs3, self.eta2, self.eta3,
                                                          self.two_body_decay, self.three_body_weight,
                                                          self.three_body_decay, self.rcut)
