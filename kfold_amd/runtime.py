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


def load_reference_weights(module, state_dict, prefix: str = "", strict: bool = True):
    """Fill a kfold_amd module from a state dict of the reference model (reference:
    ``model.load_state_dict(torch.load(..., weights_only=True))``, model/model.py:611-614).

    The hip modules keep the reference's parameter names, so this is ``load_state_dict`` on the
    entries below ``prefix`` (e.g. ``"main_stack."`` or ``"confidence_head.pairformer.blocks.0."``),
    restricted to the names the module has: a full KFold checkpoint also holds encoders, heads and
    embedders that have no hip counterpart.  With ``strict`` every parameter of the module must be
    found.  Returns the list of keys used."""
    own = module.state_dict()
    picked = {}
    for name in own:
        key = prefix + name
        if key in state_dict:
            picked[name] = state_dict[key]
    missing = [n for n in own if n not in picked]
    if strict and missing:
        raise KeyError(f"reference state dict lacks {len(missing)} entries under {prefix!r}, e.g. "
                       f"{prefix + missing[0]!r}")
    for name, value in picked.items():
        if tuple(value.shape) != tuple(own[name].shape):
            raise ValueError(f"{prefix + name}: shape {tuple(value.shape)} does not fit {tuple(own[name].shape)}")
    module.load_state_dict(picked, strict=False)
    return [prefix + n for n in picked]
