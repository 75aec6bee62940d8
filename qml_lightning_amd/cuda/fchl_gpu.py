"""Drop-in for the reference's `fchl_gpu` extension (qml_lightning/cuda/fchl_cuda.cpp:204-212).
Argument order is the reference's; the kernels there do not read the charges argument (element
types carry the information), here it only supplies the atom counts."""
import torch

from .. import ops


def _prm(species, Rs2, Rs3, eta2, eta3, two_body_decay, three_body_weight, three_body_decay, rcut):
    return ops.make_params(species.shape[0], Rs2, Rs3, eta2, eta3, two_body_decay, three_body_weight,
                           three_body_decay, rcut)


def get_element_types_gpu(coordinates, charges, natom_counts, species):
    return ops.element_types(coordinates, charges, natom_counts, species)


def get_fchl_representation(coordinates, charges, species, element_types, cell, inv_cell, blockAtomIDs, blockMolIDs,
                            neighbourlist, nneighbours, two_body_gridpoints, three_body_gridpoints, eta2, eta3,
                            two_body_decay, three_body_weight, three_body_decay, rcut):
    prm = _prm(species, two_body_gridpoints, three_body_gridpoints, eta2, eta3, two_body_decay, three_body_weight,
               three_body_decay, rcut)
    return ops.fchl_forward(coordinates, element_types, cell, inv_cell, blockAtomIDs, blockMolIDs,
                            _counts(coordinates, charges), two_body_gridpoints, three_body_gridpoints, prm,
                            neighbourlist, nneighbours)


def get_fchl_derivative(coordinates, charges, species, element_types, cell, inv_cell, blockAtomIDs, blockMolIDs,
                        neighbourlist, nneighbours, two_body_gridpoints, three_body_gridpoints, eta2, eta3,
                        two_body_decay, three_body_weight, three_body_decay, rcut):
    prm = _prm(species, two_body_gridpoints, three_body_gridpoints, eta2, eta3, two_body_decay, three_body_weight,
               three_body_decay, rcut)
    _, jac = ops.fchl_jacobian(coordinates, element_types, cell, inv_cell, blockAtomIDs, blockMolIDs,
                               _counts(coordinates, charges), two_body_gridpoints, three_body_gridpoints, prm,
                               neighbourlist, nneighbours, with_rep=False)
    return jac


def get_fchl_and_derivative(coordinates, charges, species, element_types, cell, inv_cell, blockAtomIDs, blockMolIDs,
                            neighbourlist, nneighbours, two_body_gridpoints, three_body_gridpoints, eta2, eta3,
                            two_body_decay, three_body_weight, three_body_decay, rcut, gradients):
    prm = _prm(species, two_body_gridpoints, three_body_gridpoints, eta2, eta3, two_body_decay, three_body_weight,
               three_body_decay, rcut)
    counts = _counts(coordinates, charges)
    if gradients:
        rep, jac = ops.fchl_jacobian(coordinates, element_types, cell, inv_cell, blockAtomIDs, blockMolIDs, counts,
                                     two_body_gridpoints, three_body_gridpoints, prm, neighbourlist, nneighbours)
        return [rep, jac]
    return [ops.fchl_forward(coordinates, element_types, cell, inv_cell, blockAtomIDs, blockMolIDs, counts,
                             two_body_gridpoints, three_body_gridpoints, prm, neighbourlist, nneighbours)]


def fchl_backwards(coordinates, charges, species, element_types, cell, inv_cell, blockAtomIDs, blockMolIDs,
                   neighbourlist, nneighbours, two_body_gridpoints, three_body_gridpoints, eta2, eta3, two_body_decay,
                   three_body_weight, three_body_decay, rcut, grad_in):
    prm = _prm(species, two_body_gridpoints, three_body_gridpoints, eta2, eta3, two_body_decay, three_body_weight,
               three_body_decay, rcut)
    return ops.fchl_vjp(grad_in, coordinates, element_types, cell, inv_cell, blockAtomIDs, blockMolIDs,
                        _counts(coordinates, charges), two_body_gridpoints, three_body_gridpoints, prm,
                        neighbourlist, nneighbours)


def _counts(coordinates, charges):
    """The reference's signatures carry no atom counts (its kernels only walk the neighbour list
    they are given).  Here they are recovered from the zero-padded charges (padding has charge
    0 and trails the real atoms, models/kernel.py:631-648): the count of a molecule is the index
    of its last atom with a non-zero charge, plus one, so that a call without a list, where the
    kernel finds the neighbours itself, does not take padded slots for atoms at the origin,
    and a dummy atom of charge zero INSIDE a molecule does not cut the molecule short (it gets
    element type -1 and the kernels skip it as a neighbour; the reference's kernels index out of
    bounds with such a type, fchl_cuda_kernel.cu:1732-1739)."""
    if charges.dim() == 1:
        charges = charges.unsqueeze(0)
    n = charges.shape[1]
    pos = torch.arange(1, n + 1, device=charges.device, dtype=torch.int32)
    return (pos * (charges != 0)).amax(dim=1).to(torch.int32) if n > 0 else charges.new_zeros(charges.shape[0], dtype=torch.int32)
