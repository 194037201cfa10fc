"""Backend selection with the ``hip`` value added.

Mirror of the reference's ``select_kernel_backend``
(src/kfold/utils/runtime.py:44-69): same validation and error type, one more choice.
"""

from __future__ import annotations

from . import _lib

KERNEL_BACKENDS = ("auto", "torch", "triton", "cuequiv", "hip")


def is_hip_available() -> bool:
    """True when torch is a ROCm build that sees a GPU and libkfold_hip.so loads."""
    try:
        import torch

        if getattr(torch.version, "hip", None) is None or not torch.cuda.is_available():
            return False
        _lib.lib()
        return True
    except Exception:
        return False


def select_kernel_backend(backend: str = "auto") -> str:
    """Resolve ``auto`` to ``hip`` on a ROCm GPU; validate an explicit choice."""
    if backend not in KERNEL_BACKENDS:
        raise ValueError(
            f"Unknown kernel_backend {backend!r}. "
            "Expected 'auto', 'torch', 'triton', 'cuequiv', or 'hip'.")
    if backend == "auto":
        return "hip" if is_hip_available() else "torch"
    if backend == "hip" and not is_hip_available():
        raise ValueError(
            "The hip backend is not available. It needs a ROCm build of PyTorch, a visible "
            "GPU and a built kfold_amd/libkfold_hip.so (python -m kfold_amd.build).")
    return backend
