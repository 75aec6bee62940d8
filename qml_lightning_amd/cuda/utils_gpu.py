"""Drop-in for the one function of the reference's `utils_gpu` extension that its models
use (qml_lightning/cuda/utils_cuda.cpp:26-33, called at models/kernel.py:177,188)."""
from .. import ops


def matmul_and_reduce(A, B, C):
    """C (fp64) += double(A (fp32) @ B (fp32)) with an fp32 Kahan-compensated inner sum."""
    ops.matmul_and_reduce(A, B, C)
