"""Conventions shared by the hip entry functions (same as the reference's triton wrappers)."""

from __future__ import annotations

import torch
from torch import nn


# softmax masking: the kernels give a masked key probability exactly 0 (and attend uniformly
# when every key of a row is masked), which is what the reference's finite ``-inf * (1 - mask)``
# term does in fp32 for any ``inf`` large enough that exp(-inf + logit) underflows
MIN_INF = 1e4


def check_inf(module: nn.Module) -> None:
    inf = getattr(module, "inf", 1e9)
    if not inf >= MIN_INF:
        raise NotImplementedError(
            f"The hip backend implements hard masking (inf >= {MIN_INF:g}); got inf={inf!r}")


def cache_key(parameters, x: torch.Tensor, dtype: torch.dtype) -> tuple:
    """Packed-weight cache key: device, dtype and (storage pointer, version) of every
    parameter (reference: model/primitives/triangle_multiplication.py:73-91)."""
    return (x.device.type, x.device.index, dtype) + tuple(
        value
        for p in parameters
        for value in ((None, None) if p is None else
                      (p.data_ptr(), None if torch.is_inference(p) else p._version)))


def check_inference(x: torch.Tensor, what: str) -> None:
    if torch.is_grad_enabled():
        raise RuntimeError(f"The hip {what} backend is inference-only.")
    if not x.is_cuda:
        raise RuntimeError(f"The hip {what} backend requires a ROCm GPU tensor.")


def cached_blob(module: nn.Module, attr: str, key: tuple, make):
    if getattr(module, attr + "_key", None) != key or getattr(module, attr, None) is None:
        setattr(module, attr, make())
        setattr(module, attr + "_key", key)
    return getattr(module, attr)
