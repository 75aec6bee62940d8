"""MI355X-native hot path of QML-Lightning: FCHL19 + SORF/RFF features + Z^T Z.

Importing the package registers `torch.ops.qml_lightning_fchl.*` and
`torch.ops.qml_lightning_sorf.*` (the operators the reference's TorchScript libraries
export, qml_lightning/__init__.py:13-14), implemented by the hand-written HIP library
`libqmll.so` that sits next to this file.  The library is loaded on first use; nothing
falls back to PyTorch or to the CPU when it is missing.
"""
from . import ops as _ops

_ops.register_ops()

__all__ = ["ops"]
