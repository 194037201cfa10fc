"""kfold_amd — MI355X (gfx950) backend for K-Fold's Pairformer pair-update path.

``kernel_backend="hip"`` modules with the reference's interfaces, on top of
``libkfold_hip.so`` (C ABI in ``include/kfold_hip.h``).  Nothing here falls back to another
implementation: without the built library every op raises.
"""

from .runtime import is_hip_available, select_kernel_backend  # noqa: F401

__all__ = ["select_kernel_backend", "is_hip_available"]
