"""Drop-in for the reference's `sorf_gpu` extension (qml_lightning/cuda/hadamard_cuda.cpp:111-126)."""
import torch

from .. import ops


def sorf_matrix_gpu(input, scaling):
    """[A,d] x D[T,S,d] -> [A,S*d], Hadamard-normalised only (hadamard_cuda.cpp:72-87)."""
    out = ops.sorf_forward(input, scaling, 1.0, scaling.shape[0])
    return out.view(out.shape[0], out.shape[1] * out.shape[2])


def hadamard_transform_gpu(input, dmatrix, normalisation, ntransforms):
    return ops.sorf_forward(input, dmatrix, normalisation, ntransforms)


def hadamard_transform_backwards_gpu(input, dmatrix, normalisation, ntransforms):
    return ops.sorf_adjoint(input, dmatrix, normalisation, ntransforms)


def CosFeaturesCUDA(coeffs, b, nmol, batch_indexes):
    return ops.cos_features(coeffs, b, nmol, batch_indexes)


def CosDerivativeFeaturesCUDA(grads, coeffs, b, nmol, batch_indexes):
    return ops.cos_features_backward(grads, coeffs, b, nmol, batch_indexes)


def compute_hadamard_features(sorf_matrix, bias, ordering, features):
    """features (fp64 or fp32 [nmol,F]) += sqrt(2/F) cos(sorf_matrix + bias) (hadamard_cuda.cpp:89-93)."""
    ops.cos_features(sorf_matrix, bias, features.shape[0], ordering, out=features)


def compute_partial_feature_derivatives(sorf_matrix, bias, sin_coeffs):
    ops.sin_coeffs(sorf_matrix, bias, sin_coeffs)


def compute_molecular_featurization_derivative(cos_derivs, normalisation, scaling, input_derivatives, ordering,
                                               feature_derivatives):
    ops.derivative_features(cos_derivs, normalisation, scaling, input_derivatives, ordering, feature_derivatives)


def compute_hadamard_derivative_features(sorf_matrix, normalisation, bias, scaling, input_derivatives, ordering,
                                         feature_derivatives):
    """hadamard_cuda.cpp:95-109: sin coefficients, then the full chain."""
    partial = torch.zeros(sorf_matrix.shape, dtype=torch.float64, device=sorf_matrix.device)
    ops.sin_coeffs(sorf_matrix, bias, partial)
    ops.derivative_features(partial, normalisation, scaling, input_derivatives, ordering, feature_derivatives)
