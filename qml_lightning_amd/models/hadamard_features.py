"""HadamardFeaturesModel: SORF feature model (qml_lightning/models/hadamard_features.py:13-256).

`forward(X, Z, atomIDs, molIDs, atom_counts[, cell, inv_cell])` is TorchScript-compilable
and differentiable in X.  With `fused=False` it is the reference's own operator sequence
(get_SORF_coefficients -> get_cos_features -> matmul with alpha), so a file written by
`save_jit_model` then only needs the operators the reference registers.  With
`fused=True` (default) each element goes through one kernel that never materialises the
[atoms, nfeatures] coefficients and already returns the gradient with respect to the
projected representation; the numbers are the same.
"""
from typing import Final, Optional

import numpy as np
import torch

from .. import ops
from ..cuda.sorf_gpu import compute_hadamard_features, compute_partial_feature_derivatives
from ..representations.dimensionality_reduction import project_representation
from .kernel import BaseKernel, _default_device, alpha_f32, rep_from_attribute_tree

_fused_registered = False


def _register_fused_op():
    """qml_lightning_sorf::sorf_energy(sub, D, bias, alpha, coeff_normalisation, ntransforms)
    -> per-atom energies [A]; autograd on `sub`.  Not part of the reference's operator set."""
    global _fused_registered
    if _fused_registered:
        return
    _fused_registered = True
    if ops.OPS_BACKEND == "c++":     # libqmll_torch.so has registered these operators already
        return
    lib = torch.library.Library("qml_lightning_sorf", "FRAGMENT")
    lib.define("sorf_energy(Tensor sub, Tensor D, Tensor bias, Tensor alpha, Tensor coeff_normalisation, "
               "Tensor ntransforms) -> (Tensor, Tensor)")

    def impl(sub, D, bias, alpha, cn, nt):
        e_atom = torch.empty(sub.shape[0], dtype=torch.float32, device=sub.device)
        gx = ops.sorf_energy_fused(sub, D, bias, alpha, None, ops._scalar(cn), int(nt.item()), e_atom, with_grad=True)
        return e_atom, gx

    lib.impl("sorf_energy", impl, "CompositeExplicitAutograd")

    def setup(ctx, inputs, output):
        ctx.save_for_backward(output[1])
        ctx.set_materialize_grads(False)

    def backward(ctx, g_e, g_gx):
        (gx,) = ctx.saved_tensors
        gsub = gx * g_e[:, None] if g_e is not None else None
        return gsub, None, None, None, None, None

    torch.library.register_autograd("qml_lightning_sorf::sorf_energy", backward, setup_context=setup, lib=lib)

    # all elements in one launch: x_all [N, ne*d] holds, per atom slot, the representation
    # projected with every element's reductor; the kernel picks the block of the atom's type
    lib.define("sorf_energy_typed(Tensor x_all, Tensor types, Tensor atom_slots, Tensor Dmat, Tensor bias, "
               "Tensor alpha, Tensor coeff_normalisation, Tensor ntransforms, bool with_grad) -> (Tensor, Tensor)")

    def impl_typed(x_all, types, atom_slots, Dmat, bias, alpha, cn, nt, with_grad):
        e_slots, gx = ops.sorf_energy_typed(x_all, types, atom_slots, Dmat, bias, alpha, ops._scalar(cn),
                                            int(nt.item()), with_grad=with_grad)
        if gx is None:   # energies only: the adjoint transform is skipped
            gx = torch.empty(0, dtype=torch.float32, device=x_all.device)
        return e_slots, gx

    lib.impl("sorf_energy_typed", impl_typed, "CompositeExplicitAutograd")

    def backward_typed(ctx, g_e, g_gx):
        (gx,) = ctx.saved_tensors
        if g_e is None:
            return (None,) * 9
        if gx.numel() == 0:
            raise RuntimeError("sorf_energy_typed was called with with_grad=False but a gradient is requested")
        return (gx * g_e[:, None],) + (None,) * 8

    torch.library.register_autograd("qml_lightning_sorf::sorf_energy_typed", backward_typed, setup_context=setup,
                                    lib=lib)

    # element-sorted route: sort the atoms by type, project each with its own element's
    # reductor on the matrix cores (compact [A,d]), run the fused kernel on those rows
    lib.define("sort_by_type(Tensor types, Tensor slots, int ne) -> (Tensor, Tensor)")
    lib.impl("sort_by_type", lambda types, slots, ne: ops.sort_by_type(types, slots, ne), "CompositeExplicitAutograd")
    lib.define("project_typed(Tensor rep, Tensor sorted_slots, Tensor type_offsets, Tensor reductors, Tensor types) "
               "-> Tensor")
    lib.define("project_typed_backward(Tensor gx, Tensor sorted_slots, Tensor type_offsets, Tensor reductors, "
               "Tensor types, int nslots) -> Tensor")
    lib.impl("project_typed", lambda rep, ss, off, red, types: ops.project_typed(rep, ss, off, red),
             "CompositeExplicitAutograd")
    lib.impl("project_typed_backward",
             lambda gx, ss, off, red, types, nslots: ops.project_typed_backward(gx, ss, off, red, types, nslots),
             "CompositeExplicitAutograd")

    def project_setup(ctx, inputs, output):
        rep, ss, off, red, types = inputs
        ctx.save_for_backward(ss, off, red, types)
        ctx.nslots = rep.shape[0]

    def project_backward(ctx, g):
        ss, off, red, types = ctx.saved_tensors
        g_rep = torch.ops.qml_lightning_sorf.project_typed_backward(g.contiguous(), ss, off, red, types, ctx.nslots)
        return g_rep, None, None, None, None

    torch.library.register_autograd("qml_lightning_sorf::project_typed", project_backward, setup_context=project_setup,
                                    lib=lib)

    lib.define("sorf_energy_sorted(Tensor x, Tensor type_offsets, Tensor sorted_slots, Tensor Dmat, Tensor bias, "
               "Tensor alpha, Tensor coeff_normalisation, Tensor ntransforms, int nslots, bool with_grad) "
               "-> (Tensor, Tensor)")

    def impl_sorted(x, off, ss, Dmat, bias, alpha, cn, nt, nslots, with_grad):
        e_slots, gx = ops.sorf_energy_sorted(x, off, ss, Dmat, bias, alpha, ops._scalar(cn), int(nt.item()), nslots,
                                             with_grad=with_grad)
        if gx is None:   # energies only: the adjoint transform is skipped
            gx = torch.empty(0, dtype=torch.float32, device=x.device)
        return e_slots, gx

    lib.impl("sorf_energy_sorted", impl_sorted, "CompositeExplicitAutograd")

    def setup_sorted(ctx, inputs, output):
        ctx.save_for_backward(output[1], inputs[2])
        ctx.set_materialize_grads(False)

    def backward_sorted(ctx, g_e, g_gx):
        gx, ss = ctx.saved_tensors
        if g_e is None:
            return (None,) * 10
        if gx.numel() == 0 and ss.numel() != 0:
            raise RuntimeError("sorf_energy_sorted was called with with_grad=False but a gradient is requested")
        return (gx * g_e.index_select(0, ss.long())[:, None],) + (None,) * 9

    torch.library.register_autograd("qml_lightning_sorf::sorf_energy_sorted", backward_sorted,
                                    setup_context=setup_sorted, lib=lib)

    # random Fourier features on the same element-sorted rows
    lib.define("rff_energy_sorted(Tensor x, Tensor type_offsets, Tensor sorted_slots, Tensor W, Tensor b, "
               "Tensor alpha, int nslots, bool with_grad) -> (Tensor, Tensor)")

    def impl_rff(x, off, ss, W, b, alpha, nslots, with_grad):
        e_slots, gx = ops.rff_energy_sorted(x, off, ss, W, b, alpha, nslots, with_grad=with_grad)
        if gx is None:
            gx = torch.empty(0, dtype=torch.float32, device=x.device)
        return e_slots, gx

    lib.impl("rff_energy_sorted", impl_rff, "CompositeExplicitAutograd")

    def backward_rff(ctx, g_e, g_gx):
        gx, ss = ctx.saved_tensors
        if g_e is None:
            return (None,) * 8
        if gx.numel() == 0 and ss.numel() != 0:
            raise RuntimeError("rff_energy_sorted was called with with_grad=False but a gradient is requested")
        return (gx * g_e.index_select(0, ss.long())[:, None],) + (None,) * 7

    torch.library.register_autograd("qml_lightning_sorf::rff_energy_sorted", backward_rff, setup_context=setup_sorted,
                                    lib=lib)
    # the whole fused chain as one operator: one dispatch and one autograd node per evaluation
    lib.define("fchl_sorf_energy(%s, Tensor reductors, Tensor Dmat, Tensor bias, Tensor alpha, "
               "Tensor coeff_normalisation, Tensor ntransforms, Tensor model_species, bool with_grad) "
               "-> (Tensor, Tensor)" % ops._FCHL_SIG)

    def check_model(species, model_species, reductors, R):
        """The model's element list (hadamard_features.py:99-107 selects atoms with Z == e over it) may
        differ from the representation's species; its length must match the reductors."""
        if reductors.dim() != 3 or reductors.shape[1] != R:
            raise RuntimeError("fchl_sorf_energy: reductors are %s, the representation has %d entries per atom"
                               % (tuple(reductors.shape), R))
        if model_species.numel() == 0:
            if reductors.shape[0] != species.shape[0]:
                raise RuntimeError("fchl_sorf_energy: the model has %d elements, the representation %d species, and "
                                   "no model species were given" % (reductors.shape[0], species.shape[0]))
        elif model_species.numel() != reductors.shape[0]:
            raise RuntimeError("fchl_sorf_energy: %d model species for %d reductors"
                               % (model_species.numel(), reductors.shape[0]))

    def impl_chain(X, Z, species, atomIDs, molIDs, atom_counts, cell, inv_cell, Rs2, Rs3, eta2, eta3, two_body_decay,
                   three_body_weight, three_body_decay, rcut, reductors, Dmat, bias, alpha, cn, nt, model_species,
                   with_grad, gscale=1.0):
        Xb, Zb = ops._batched(X, Z)
        B, n = Zb.shape
        nslots = B * n
        prm = ops.make_params(species.shape[0], Rs2, Rs3, eta2, eta3, two_body_decay, three_body_weight,
                              three_body_decay, rcut)
        check_model(species, model_species, reductors, ops.repsize(prm))
        # element indices, the sort by the model's element and the zero fill of what the chain adds into
        # (per-slot energies, then dE/dX): one launch for a small batch
        types, stypes, ss, off, zeroed = ops.prepare_batch(Zb, atom_counts, species, atomIDs, molIDs, model_species,
                                                           (4 if with_grad else 1) * nslots)
        cell_ = cell if cell.numel() > 0 else None
        inv_cell_ = inv_cell if inv_cell.numel() > 0 else None
        fargs = (Xb, types, cell_, inv_cell_, atomIDs, molIDs, atom_counts, Rs2, Rs3, prm)
        rep = ops.fchl_forward(*fargs, zero_fill=False)
        x = ops.project_typed(rep.view(nslots, -1), ss, off, reductors)
        e_slots, gx = ops.sorf_energy_sorted(x, off, ss, Dmat, bias, alpha, ops._scalar(cn), int(nt.item()), nslots,
                                             with_grad=with_grad, e_zeroed=zeroed[:nslots])
        if not with_grad:
            return ops.molecule_sums(e_slots, B, n), torch.empty(0, dtype=torch.float32, device=X.device)
        g_rep, energies = ops.project_typed_backward_sums(gx, ss, off, reductors, stypes, nslots, e_slots, B, n)
        return energies, ops.fchl_vjp(g_rep.view(rep.shape), *fargs, out=zeroed[nslots:].view(B, n, 3), scale=gscale)

    lib.impl("fchl_sorf_energy", impl_chain, "CompositeExplicitAutograd")

    # the same chain with random Fourier features: W in place of the diagonals, b in place of the bias
    lib.define("fchl_rff_energy(%s, Tensor reductors, Tensor W, Tensor b, Tensor alpha, Tensor model_species, "
               "bool with_grad) -> (Tensor, Tensor)" % ops._FCHL_SIG)

    def impl_chain_rff(X, Z, species, atomIDs, molIDs, atom_counts, cell, inv_cell, Rs2, Rs3, eta2, eta3,
                       two_body_decay, three_body_weight, three_body_decay, rcut, reductors, W, b, alpha,
                       model_species, with_grad, gscale=1.0):
        Xb, Zb = ops._batched(X, Z)
        B, n = Zb.shape
        nslots = B * n
        prm = ops.make_params(species.shape[0], Rs2, Rs3, eta2, eta3, two_body_decay, three_body_weight,
                              three_body_decay, rcut)
        check_model(species, model_species, reductors, ops.repsize(prm))
        types, stypes, ss, off, zeroed = ops.prepare_batch(Zb, atom_counts, species, atomIDs, molIDs, model_species,
                                                           (4 if with_grad else 1) * nslots)
        fargs = (Xb, types, cell if cell.numel() > 0 else None, inv_cell if inv_cell.numel() > 0 else None, atomIDs,
                 molIDs, atom_counts, Rs2, Rs3, prm)
        rep = ops.fchl_forward(*fargs, zero_fill=False)
        x = ops.project_typed(rep.view(nslots, -1), ss, off, reductors)
        e_slots, gx = ops.rff_energy_sorted(x, off, ss, W, b, alpha, nslots, with_grad=with_grad,
                                            e_zeroed=zeroed[:nslots])
        if not with_grad:
            return ops.molecule_sums(e_slots, B, n), torch.empty(0, dtype=torch.float32, device=X.device)
        g_rep, energies = ops.project_typed_backward_sums(gx, ss, off, reductors, stypes, nslots, e_slots, B, n)
        return energies, ops.fchl_vjp(g_rep.view(rep.shape), *fargs, out=zeroed[nslots:].view(B, n, 3), scale=gscale)

    lib.impl("fchl_rff_energy", impl_chain_rff, "CompositeExplicitAutograd")

    # (energies, forces = -dE/dX) with no autograd graph: the sign is applied inside the last kernel of the chain
    def no_graph(X, who):
        if torch.is_grad_enabled() and X.requires_grad:
            raise RuntimeError(who + " builds no autograd graph: call it under no_grad, or use the _energy operator "
                               "for a differentiable result")

    def impl_forces(*args):
        no_graph(args[0], "fchl_sorf_forces")
        with torch.no_grad():
            e, F = impl_chain(*args, True, gscale=-1.0)
        return e, (F.squeeze(0) if args[0].dim() == 2 else F)

    def impl_forces_rff(*args):
        no_graph(args[0], "fchl_rff_forces")
        with torch.no_grad():
            e, F = impl_chain_rff(*args, True, gscale=-1.0)
        return e, (F.squeeze(0) if args[0].dim() == 2 else F)

    lib.define("fchl_sorf_forces(%s, Tensor reductors, Tensor Dmat, Tensor bias, Tensor alpha, "
               "Tensor coeff_normalisation, Tensor ntransforms, Tensor model_species) -> (Tensor, Tensor)" % ops._FCHL_SIG)
    lib.impl("fchl_sorf_forces", impl_forces, "CompositeExplicitAutograd")
    lib.define("fchl_rff_forces(%s, Tensor reductors, Tensor W, Tensor b, Tensor alpha, Tensor model_species) "
               "-> (Tensor, Tensor)" % ops._FCHL_SIG)
    lib.impl("fchl_rff_forces", impl_forces_rff, "CompositeExplicitAutograd")

    def setup_chain(ctx, inputs, output):
        ctx.save_for_backward(output[1])
        ctx.xdim = inputs[0].dim()
        ctx.set_materialize_grads(False)

    def backward_chain(ctx, g_e, g_gx):
        (gX,) = ctx.saved_tensors
        if g_e is None:
            return (None,) * 24
        if gX.dim() != 3:
            raise RuntimeError("fchl_sorf_energy was called with with_grad=False but a gradient is requested")
        g = gX * g_e.reshape(-1, 1, 1)
        return (g.squeeze(0) if ctx.xdim == 2 else g,) + (None,) * 23

    torch.library.register_autograd("qml_lightning_sorf::fchl_sorf_energy", backward_chain, setup_context=setup_chain,
                                    lib=lib)

    def backward_chain_rff(ctx, g_e, g_gx):
        (gX,) = ctx.saved_tensors
        if g_e is None:
            return (None,) * 22
        if gX.dim() != 3:
            raise RuntimeError("fchl_rff_energy was called with with_grad=False but a gradient is requested")
        g = gX * g_e.reshape(-1, 1, 1)
        return (g.squeeze(0) if ctx.xdim == 2 else g,) + (None,) * 21

    torch.library.register_autograd("qml_lightning_sorf::fchl_rff_energy", backward_chain_rff,
                                    setup_context=setup_chain, lib=lib)
    ops._libs.append(lib)


_register_fused_op()


def model_species_for_sort(species, rep):
    """What the one-operator predict chain gets as `model_species`: the model's element list
    when it differs from the representation's species list (a subset, another order), else an
    empty tensor, which lets the chain reuse the representation's element types."""
    if rep is not None and tuple(rep.species.shape) == tuple(species.shape) and bool((rep.species.cpu() == species.cpu()).all()):
        return torch.empty(0, dtype=torch.float32, device=species.device)
    return species


_NO_CELLS = {}
_NORMALISATION = {}


def _no_cells(device):
    """The empty [0,3,3] tensor that says "no periodic images", one per device (a single molecule's
    step is as long as its host side: nothing is built per call that can be kept)."""
    t = _NO_CELLS.get(device)
    if t is None:
        t = _NO_CELLS[device] = torch.empty(0, 3, 3, device=device)
    return t


def _normalisation_tensor(npcas, sigma):
    key = (int(npcas), float(sigma))
    t = _NORMALISATION.get(key)
    if t is None:
        if len(_NORMALISATION) > 256:
            _NORMALISATION.clear()
        t = _NORMALISATION[key] = torch.tensor(float(np.sqrt(np.float32(npcas)) / np.float32(sigma)))
    return t


@torch.jit.ignore
def _eager_constants(model, device: torch.device, cell: Optional[torch.Tensor], inv_cell: Optional[torch.Tensor]):
    if cell is None:
        cell = _no_cells(device)
    if inv_cell is None:
        inv_cell = _no_cells(device)
    if isinstance(model.sigma, float):
        cn = _normalisation_tensor(model.npcas, model.sigma)
    else:
        cn = torch.sqrt(torch.tensor(model.npcas)) / model.sigma
    return cell, inv_cell, cn, alpha_f32(model)


class HadamardFeaturesModel(BaseKernel, torch.nn.Module):

    fused: Final[bool]
    separate_ops: Final[bool]

    def __init__(self, rep=None, elements=np.array([1, 6, 7, 8]), ntransforms=2, sigma=3.0, llambda=1e-11, npcas=128,
                 nbatch_train=64, nbatch_test=64, nstacks=32, fused=True, separate_ops=False):
        torch.nn.Module.__init__(self)
        BaseKernel.__init__(self, rep, npcas, elements, sigma, llambda)
        self.device = _default_device()
        self.ntransforms = torch.tensor(ntransforms)
        self.nstacks = nstacks
        self.nbatch_train = nbatch_train
        self.nbatch_test = nbatch_test
        self.species = torch.from_numpy(np.asarray(elements)).float().to(self.device)
        self.sort_species = model_species_for_sort(self.species, rep)
        self.npcas = npcas
        self.fused = fused
        self.separate_ops = separate_ops   # fused route as five operators (one node each) instead of one
        self._pending_derivative_features = []
        self.Dmat = torch.zeros((len(elements), ntransforms, nstacks, npcas), dtype=torch.float32, device=self.device)
        self.get_SORF_diagonals(elements, ntransforms, nstacks, npcas)
        self.bias = torch.zeros((len(elements), self.nfeatures()), dtype=torch.float32, device=self.device)
        self.get_bias(elements, nstacks * npcas)
        self.is_trained = False
        self.alpha = torch.zeros(self.nfeatures(), device=self.device, dtype=torch.float)

    @torch.jit.unused
    def get_SORF_diagonals(self, elements, ntransforms, nstacks, npcas):
        """Rademacher diagonals per element (hadamard_features.py:44-53)."""
        for e in elements:
            D = np.random.uniform(-1, 1, (ntransforms, nstacks, npcas))
            D = np.where(D > 0.0, 1.0, -1.0)
            self.Dmat[self.element2index[int(e)]] = torch.from_numpy(D).float().to(self.device)

    @torch.jit.unused
    def get_bias(self, elements, nfeatures):
        """b ~ U(0, 2 pi) per element (hadamard_features.py:55-61)."""
        for e in elements:
            v = np.random.uniform(0.0, 1.0, [nfeatures]) * 2.0 * np.pi
            self.bias[self.element2index[int(e)]] = torch.from_numpy(v).float().to(self.device)

    def nfeatures(self):
        return self.npcas * self.nstacks

    @torch.jit.unused
    def calculate_features(self, representation, element, indexes, feature_matrix, grad=None,
                           derivative_features=None):
        """Add one element's cos features (and force features) into the fp64 batch
        matrices (hadamard_features.py:66-80)."""
        coeff_normalisation = np.sqrt(representation.shape[1]) / self.sigma
        element_idx = self.element2index[int(element)]
        coeffs = ops.sorf_forward(representation, self.Dmat[element_idx], coeff_normalisation, int(self.ntransforms))
        coeffs = coeffs.view(coeffs.shape[0], -1)
        compute_hadamard_features(coeffs, self.bias[element_idx], indexes, feature_matrix)
        if derivative_features is not None and grad is not None:
            cos_derivs = torch.empty(coeffs.shape, device=coeffs.device, dtype=torch.float64)
            compute_partial_feature_derivatives(coeffs, self.bias[element_idx], cos_derivs)
            if self._queue_force_rows:
                # all elements go through ONE launch once the batch's loop over elements is done
                # (finish_features): every element of the force-feature block is then read and
                # written once instead of once per element and atom chunk
                self._pending_derivative_features.append((cos_derivs, self.Dmat[element_idx], grad, indexes))
                return
            # `indexes` comes from a molecule-major gather, so the atomic-free kernel applies
            ops.derivative_features(cos_derivs, coeff_normalisation, self.Dmat[element_idx], grad, indexes,
                                    derivative_features, molecule_major=True)

    @torch.jit.unused
    def writes_force_rows(self):
        return 64 <= self.npcas <= 256 and len(self.elements) <= 8

    @torch.jit.unused
    def finish_features(self, derivative_features=None, overwrite=False):
        """Force-feature rows of the elements queued by calculate_features, in one launch."""
        pending, self._pending_derivative_features = self._pending_derivative_features, []
        if derivative_features is not None and (pending or overwrite):
            ops.derivative_features_typed(pending, float(np.sqrt(self.npcas) / self.sigma), derivative_features,
                                          overwrite=overwrite)

    def forward(self, X, Z, atomIDs, molIDs, atom_counts, cell: Optional[torch.Tensor] = None,
                inv_cell: Optional[torch.Tensor] = None):
        """Total energies [B] (fp32), differentiable in X (hadamard_features.py:82-123)."""
        if torch.jit.is_scripting():
            if cell is None:
                cell = torch.empty(0, 3, 3, device=X.device)
            if inv_cell is None:
                inv_cell = torch.empty(0, 3, 3, device=X.device)
            coeff_normalisation = torch.sqrt(torch.tensor(self.npcas)) / self.sigma
            # the fused operators take alpha as it is stored (fp64) and keep its fp32 form per tensor
            # version; the reference's route below converts it where it contracts with it
            alpha = self.alpha
        else:
            # the same values without building them per call (a single molecule's step is as long as its
            # host side): the empty cell tensor and the normalisation are kept, alpha converted once per value
            cell, inv_cell, coeff_normalisation, alpha = _eager_constants(self, X.device, cell, inv_cell)
        assert X.is_cuda, "X tensor must reside on GPU"
        assert Z.is_cuda, "Z tensor must reside on GPU"
        assert atomIDs.is_cuda, "atomIDs tensor must reside on GPU"
        assert molIDs.is_cuda, "molIDs tensor must reside on GPU"
        assert atom_counts.is_cuda, "atom_counts tensor must reside on GPU"
        assert cell.is_cuda, "cell tensor must reside on GPU"
        assert inv_cell.is_cuda, "inv_cell tensor must reside on GPU"

        if self.fused and not self.separate_ops:
            # the whole chain below (representation, sort by element, projection, SORF + cos +
            # energy and, for a gradient, its backward) as ONE operator and one autograd node
            energies, _ = torch.ops.qml_lightning_sorf.fchl_sorf_energy(
                X, Z, self.rep.species, atomIDs, molIDs, atom_counts, cell, inv_cell, self.rep.Rs2, self.rep.Rs3,
                self.rep.eta2, self.rep.eta3, self.rep.two_body_decay, self.rep.three_body_weight,
                self.rep.three_body_decay, self.rep.rcut, self.reductors, self.Dmat, self.bias, alpha,
                coeff_normalisation, self.ntransforms, self.sort_species, X.requires_grad)
            return energies

        torch_rep = self.rep.forward(X, Z, atomIDs, molIDs, atom_counts, cell, inv_cell)

        if self.fused:
            # the atoms are sorted by element on the device (no host round trip for sizes);
            # one matrix-core kernel projects each with its own element's reductor into compact
            # rows, and one kernel runs SORF + cos + energy (+ gradient) on those rows
            nslots = X.shape[0] * X.shape[1]
            flat_rep = torch_rep.view(nslots, torch_rep.shape[2])
            types = torch.ops.qml_lightning_fchl.get_element_types(X, Z, atom_counts, self.species).view(-1)
            slots = molIDs * X.shape[1] + atomIDs
            sorted_slots, type_offsets = torch.ops.qml_lightning_sorf.sort_by_type(types, slots,
                                                                                   self.reductors.shape[0])
            x = torch.ops.qml_lightning_sorf.project_typed(flat_rep, sorted_slots, type_offsets, self.reductors, types)
            e_slots, _ = torch.ops.qml_lightning_sorf.sorf_energy_sorted(x, type_offsets, sorted_slots, self.Dmat,
                                                                         self.bias, alpha, coeff_normalisation,
                                                                         self.ntransforms, nslots, x.requires_grad)
            return e_slots.view(X.shape[0], X.shape[1]).sum(dim=1)

        # The reference's operator sequence (hadamard_features.py:99-121) with nothing but its own
        # operators and plain torch, so a file saved from here loads wherever the reference's
        # libraries are.  Each element's atoms are looked up ONCE (one host round trip for the
        # count) and gathered with index_select, whose backward is an index_add: the boolean-mask
        # forms `rep[Z == e]` and `where(Z == e)` of the reference each search again, forward and
        # backward (nine round trips per step for three elements instead of three).
        nmol, natoms_max = torch_rep.shape[0], torch_rep.shape[1]      # [1, n] for one unbatched molecule
        Ztest = torch.zeros(nmol, self.nfeatures(), device=X.device, dtype=torch.float32)
        flat_rep = torch_rep.view(nmol * natoms_max, torch_rep.shape[2])
        flat_charges = Z.int().view(-1)
        for e in self.elements:
            element_idx = self.element2index[e]
            atom_rows = torch.nonzero(flat_charges == e.item())[:, 0]      # ascending: molecule-major
            if atom_rows.shape[0] == 0:
                continue
            batch_indexes = torch.div(atom_rows, natoms_max, rounding_mode='floor').type(torch.int)
            sub = flat_rep.index_select(0, atom_rows)
            sub = project_representation(sub, self.reductors[element_idx])
            coeffs = torch.ops.qml_lightning_sorf.get_SORF_coefficients(sub, self.Dmat[element_idx],
                                                                        coeff_normalisation, self.ntransforms)
            coeffs = coeffs.view(coeffs.shape[0], coeffs.shape[1] * coeffs.shape[2])
            features = torch.ops.qml_lightning_sorf.get_cos_features(coeffs, self.bias[element_idx],
                                                                     torch.tensor(nmol), batch_indexes)
            Ztest = Ztest + features
        return torch.matmul(Ztest, alpha.float())

    @torch.jit.unused
    def energies_and_forces(self, coordinates, charges, atomIDs, molIDs, natom_counts, cells=None, inv_cells=None,
                            forces=True):
        """(energies [B], forces [B,n,3] or None) for device tensors through the fused route,
        asynchronously on the current stream.  The fused kernel returns dE/dx itself, so the
        forces need no autograd graph: same numbers as `forward` + `autograd.grad`."""
        # one call of the operator that runs the whole chain (what `forward` dispatches to), outside
        # autograd: it returns the energies and dE/dX
        if cells is None or inv_cells is None:
            cells = inv_cells = _no_cells(coordinates.device)
        if isinstance(self.sigma, float):       # sqrt(npcas) / sigma in fp32, as the tensor expression gives it
            coeff_normalisation = _normalisation_tensor(self.npcas, self.sigma)
        else:
            coeff_normalisation = torch.sqrt(torch.tensor(self.npcas)) / self.sigma
        rep = self.rep
        with torch.no_grad():
            if forces:      # energies and -dE/dX from one operator, the sign applied in its last kernel
                return torch.ops.qml_lightning_sorf.fchl_sorf_forces(
                    coordinates, charges, rep.species, atomIDs, molIDs, natom_counts, cells, inv_cells, rep.Rs2, rep.Rs3,
                    rep.eta2, rep.eta3, rep.two_body_decay, rep.three_body_weight, rep.three_body_decay, rep.rcut,
                    self.reductors, self.Dmat, self.bias, alpha_f32(self), coeff_normalisation, self.ntransforms,
                    self.sort_species)
            energies, _ = torch.ops.qml_lightning_sorf.fchl_sorf_energy(
                coordinates, charges, rep.species, atomIDs, molIDs, natom_counts, cells, inv_cells, rep.Rs2, rep.Rs3,
                rep.eta2, rep.eta3, rep.two_body_decay, rep.three_body_weight, rep.three_body_decay, rep.rcut,
                self.reductors, self.Dmat, self.bias, alpha_f32(self), coeff_normalisation, self.ntransforms,
                self.sort_species, False)
        return energies, None

    @torch.jit.unused
    def predict_opt(self, coordinates, charges, atomIDs, molIDs, natom_counts, cells=None, inv_cells=None,
                    forces=True, print_info=False, profiler=False):
        """Energies (and forces = -dE/dX by autograd) for tensors already on the device
        (hadamard_features.py:125-179)."""
        if self.is_trained is False:
            raise RuntimeError("Error: must train the model first by calling train()!")
        if self.fused and not profiler:
            start = torch.cuda.Event(enable_timing=True)
            end = torch.cuda.Event(enable_timing=True)
            start.record()
            result = self.energies_and_forces(coordinates, charges, atomIDs, molIDs, natom_counts, cells, inv_cells,
                                              forces=forces)
            end.record()
            torch.cuda.synchronize()
            if print_info:
                print("prediction for", coordinates.shape[0], "molecules time: ", start.elapsed_time(end), "ms")
            return result if forces else result[0]
        with torch.autograd.profiler.profile(enabled=profiler, use_device='cuda', with_stack=True) as prof:
            start = torch.cuda.Event(enable_timing=True)
            end = torch.cuda.Event(enable_timing=True)
            start.record()
            if forces:
                coordinates.requires_grad = True
            total_energies = self.forward(coordinates, charges, atomIDs, molIDs, natom_counts, cells, inv_cells)
            if forces:
                forces_torch, = torch.autograd.grad(-total_energies.sum(), coordinates)
            end.record()
            torch.cuda.synchronize()
        if print_info:
            print("prediction for", coordinates.shape[0], "molecules time: ", start.elapsed_time(end), "ms")
        result = (total_energies, forces_torch) if forces else total_energies
        if profiler:
            result = (result,) + (prof,)
        return result

    @torch.jit.unused
    def predict(self, X, Z, max_natoms, cells=None, inv_cells=None, forces=True, print_info=False, profiler=False):
        """Batched predict from lists of numpy arrays (hadamard_features.py:181-251)."""
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        start.record()
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
                                          data['natom_counts'], data['cells'], data['inv_cells'], forces=forces,
                                          print_info=False, profiler=False)
            if forces:
                predict_energies[sl] = result[0].detach()
                n = result[1].shape[1]
                # padded slots carry exactly zero force, so the padded block can be copied whole
                predict_forces[sl, :n] = result[1]
            else:
                predict_energies[sl] = result.detach()
        end.record()
        torch.cuda.synchronize()
        if print_info:
            print("prediction for", len(X), "molecules time: ", start.elapsed_time(end), "ms")
        if forces:
            return (predict_energies, predict_forces)
        return predict_energies

    @classmethod
    def from_reference_file(cls, file_name, fused=True, separate_ops=False):
        """A HadamardFeaturesModel holding the weights of a model file written by
        `save_jit_model` (hadamard_features.py:253-255 of the reference): by the reference
        itself or by this class.  The archive is read as data (attribute tree walked opcode by
        opcode, storages through numpy): nothing in it is unpickled or executed, no operator
        library and no GPU are needed to open it.  The result predicts through the fused route
        (or, with `fused=False`, the reference's operator sequence) and can be trained further
        or saved again."""
        from ..utils import model_files
        tree = model_files.read_attribute_tree(file_name)
        if not str(tree.get("__class__", "")).endswith("HadamardFeaturesModel"):
            raise ValueError("%s holds a %r, not a HadamardFeaturesModel" % (file_name, tree.get("__class__")))
        rep = rep_from_attribute_tree(tree["rep"])
        model = cls(rep=rep, elements=np.asarray(tree["elements"], dtype=np.int64),
                    ntransforms=int(tree["ntransforms"]), sigma=float(tree["sigma"]), llambda=float(tree["llambda"]),
                    npcas=int(tree["npcas"]), nbatch_train=int(tree["nbatch_train"]),
                    nbatch_test=int(tree["nbatch_test"]), nstacks=int(tree["nstacks"]), fused=fused,
                    separate_ops=separate_ops)
        model._fill_from_attribute_tree(tree, {"Dmat": torch.float32, "bias": torch.float32})
        if not bool(((model.Dmat == 1) | (model.Dmat == -1)).all()):
            raise ValueError("%s: the SORF diagonals are not all +-1" % file_name)
        return model

    @torch.jit.unused
    def save_jit_model(self, file_name='model_sorf.pt'):
        script = torch.jit.script(self)
        script.save(file_name)
