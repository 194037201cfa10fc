"""Parameter holders with the reference's names (primitives/normalization.py:22,
primitives/linear.py:22,110).  They own parameters only; the arithmetic of the hip backend
lives in the fused kernels, which read these parameters through the packed-weight cache."""

from __future__ import annotations

import torch
from torch import nn


class LayerNorm(nn.Module):
    def __init__(self, normalized_shape: int, create_scale: bool = True,
                 create_offset: bool = True, eps: float = 1e-5):
        super().__init__()
        self.normalized_shape = normalized_shape
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(normalized_shape)) if create_scale else None
        self.bias = nn.Parameter(torch.zeros(normalized_shape)) if create_offset else None


class Linear(nn.Module):
    """Weight is [out_features, in_features]; ``init`` keeps the reference's rule that
    "gating"/"final"/"zero" start at zero and everything else is drawn by the caller."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True,
                 init: str = "default"):
        super().__init__()
        self.weight = nn.Parameter(torch.zeros(out_features, in_features))
        if bias:
            self.bias = nn.Parameter(torch.zeros(out_features))
        else:
            self.register_parameter("bias", None)
        if init not in ("gating", "final", "zero"):
            # LeCun-normal scale like the reference's "default"; benchmark configs re-draw
            with torch.no_grad():
                std = in_features ** -0.5
                nn.init.trunc_normal_(self.weight, 0.0, std, -2 * std, 2 * std)


class LinearNoBias(Linear):
    def __init__(self, in_features: int, out_features: int, init: str = "default"):
        super().__init__(in_features, out_features, bias=False, init=init)
