"""Drop-in for the reference's `rff_gpu` extension (qml_lightning/cuda/random_features.cpp:35-39)."""
from .. import ops


def get_rff(input, sampling_matrix, bias, ordering, features):
    ops.rff_features(input, sampling_matrix, bias, ordering, features)


def get_rff_derivatives(input, grad, sampling_matrix, bias, ordering, feature_derivatives):
    ops.rff_derivative_features(input, grad, sampling_matrix, bias, ordering, feature_derivatives)
