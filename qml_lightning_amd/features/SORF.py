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
