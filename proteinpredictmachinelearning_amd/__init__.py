"""MI355X (gfx950) backend for the reference's matrix-multiplication graph op.

``ops`` mirrors the reference's operator interface on device tensors; ``cabi`` is the raw binding
of ``include/ppml_hip.h``.  Everything computes in hand-written HIP kernels; nothing falls back to
the CPU.
"""
from . import cabi  # noqa: F401

__all__ = ["cabi", "ops"]


def __getattr__(name):
    if name == "ops":
        import importlib

        return importlib.import_module(".ops", __name__)
    raise AttributeError(name)
