"""Drop-in for the reference's `pairlist_gpu` extension (qml_lightning/cuda/pairlist_cuda.cpp:67-72)."""
from .. import ops


def get_num_neighbours_gpu(coordinates, natoms, rcut, lattice_vecs=None, inv_lattice_vecs=None):
    """int32 [B, max_atoms] neighbour counts (pairlist_cuda.cpp:21-37)."""
    return ops.num_neighbours(coordinates, natoms, rcut, lattice_vecs, inv_lattice_vecs)


def get_neighbour_list_gpu(coordinates, natoms, max_neighbours, rcut, lattice_vecs=None, inv_lattice_vecs=None):
    """int32 [B, max_atoms, max_neighbours], ascending j, -1 padded (pairlist_cuda.cpp:47-65)."""
    return ops.neighbour_list(coordinates, natoms, max_neighbours, rcut, lattice_vecs, inv_lattice_vecs)


def safe_fill_gpu(pairlist):
    """Fill with -1 in place (pairlist_cuda.cpp:39-45)."""
    pairlist.fill_(-1)
