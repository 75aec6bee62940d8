"""Autograd wrappers of the SORF transform and the cos features
(qml_lightning/features/SORF.py:15-72)."""
import torch

from ..cuda import sorf_gpu


class SORFTransformCuda(torch.autograd.Function):
    """coefficients = normalisation * [H D]^T-chain u, differentiable in u."""

    @staticmethod
    def forward(ctx, u, d, coeff_normalisation, ntransforms):
        ctx.save_for_backward(d)
        ctx.coeff_normalisation = coeff_normalisation
        ctx.ntransforms = ntransforms
        return sorf_gpu.hadamard_transform_gpu(u, d, coeff_normalisation, ntransforms)

    @staticmethod
    def backward(ctx, grad):
        d = ctx.saved_tensors[0]
        grads = sorf_gpu.hadamard_transform_backwards_gpu(grad.contiguous(), d, ctx.coeff_normalisation, ctx.ntransforms)
        return grads, None, None, None


class CosFeatures(torch.autograd.Function):
    """Z[mol] = sum_atoms sqrt(2/F) cos(coeffs + b), differentiable in coeffs."""

    @staticmethod
    def forward(ctx, coeffs, b, nmol, batch_indexes):
        ctx.save_for_backward(coeffs, b, batch_indexes)
        ctx.nmol = nmol
        return sorf_gpu.CosFeaturesCUDA(coeffs, b, nmol, batch_indexes)

    @staticmethod
    def backward(ctx, grad):
        coeffs, b, batch_indexes = ctx.saved_tensors
        grads = sorf_gpu.CosDerivativeFeaturesCUDA(grad.contiguous(), coeffs, b, ctx.nmol, batch_indexes)
        return grads, None, None, None


# ---- module-level helpers of the reference's features/SORF.py ----------------------------------
# The models draw their own diagonals and biases (models/hadamard_features.py); these free
# functions are the older dictionary-per-element interface (features/SORF.py:83-152).

def _device():
    return torch.device("cuda:0")


def get_SORF_diagonals(elements, ntransforms, nstacks, npcas):
    """{element: D f32 [ntransforms, nstacks, npcas] of +-1} from numpy's global generator
    (features/SORF.py:83-95)."""
    import numpy as np
    out = {}
    for e in elements:
        draw = np.random.uniform(-1, 1, (ntransforms, nstacks, npcas))
        out[e] = torch.from_numpy(np.where(draw > 0.0, 1.0, -1.0)).float().to(_device())
    return out


def get_bias(elements, nfeatures):
    """{element: b f32 [nfeatures] ~ U(0, 2 pi)} (features/SORF.py:98-106)."""
    import numpy as np
    out = {}
    for e in elements:
        out[e] = torch.from_numpy(np.random.uniform(0.0, 1.0, [nfeatures]) * 2.0 * np.pi).float().to(_device())
    return out


def _timed(label, print_timings, fn):
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    out = fn()
    end.record()
    torch.cuda.synchronize()
    if print_timings:
        print(label, start.elapsed_time(end), "ms")
    return out


def get_SORF_coefficients(input_rep, diagonals, normalization, print_timings=False):
    """normalization * (Hadamard-normalised transform chain of input_rep) as [A, S*d]
    (features/SORF.py:109-124)."""
    return _timed("SORF coefficients time: ", print_timings,
                  lambda: normalization * sorf_gpu.sorf_matrix_gpu(input_rep, diagonals))


def get_features(coeffs, bias, batch_indexes, batch_num, print_timings=False):
    """fp64 [batch_num, F] cos features summed per molecule (features/SORF.py:127-141; the
    extension function the reference names there is not among the ones it exports, so this
    follows compute_hadamard_features, hadamard_cuda.cpp:89-93)."""
    def run():
        features = torch.zeros(batch_num, coeffs.shape[1], dtype=torch.float64, device=coeffs.device)
        sorf_gpu.compute_hadamard_features(coeffs, bias, batch_indexes, features)
        return features
    return _timed("features time: ", print_timings, run)


def get_feature_derivatives(coeffs, bias, diagonals, input_grad, batch_indexes, batch_num, normalization,
                            print_timings=False):
    """fp64 [batch_num, n, 3, F] force-feature rows times `normalization` (features/SORF.py:144-159;
    as above, through compute_hadamard_derivative_features, hadamard_cuda.cpp:95-109)."""
    def run():
        G = torch.zeros(batch_num, input_grad.shape[1], 3, coeffs.shape[1], dtype=torch.float64, device=coeffs.device)
        sorf_gpu.compute_hadamard_derivative_features(coeffs, 1.0, bias, diagonals, input_grad, batch_indexes, G)
        return normalization * G
    return _timed("feature derivatives time: ", print_timings, run)
