"""Counterpart of the reference's qml_lightning/torchscript/setup.py: importing it makes
the `qml_lightning_fchl` / `qml_lightning_sorf` operators available to `torch.jit.load`.
Here they are registered by importing the package; no environment variable is needed."""
import qml_lightning_amd  # noqa: F401  (registers the operators)
