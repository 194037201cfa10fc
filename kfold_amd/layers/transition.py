"""Transition (SwiGLU MLP), ``hip`` backend.

Mirror of the reference's ``Transition`` (src/kfold/model/layers/folding/transition.py:20-68)
and ``SwiGLU`` (model/primitives/activation.py:20-29): same constructor and parameter names
(``layernorm``, ``swiglu.linear``, ``linear_out``).
"""

from __future__ import annotations

import torch
from torch import nn

from .. import ops
from ..primitives._common import cache_key, cached_blob, check_inference
from ..primitives.layers import LayerNorm, LinearNoBias


def _parameters(module: nn.Module):
    return (module.layernorm.weight, module.layernorm.bias, module.swiglu.linear.weight,
            module.linear_out.weight)


@torch.compiler.disable
def hip_transition(module: nn.Module, x: torch.Tensor, residual: torch.Tensor | None = None,
                   mask: torch.Tensor | None = None, out: torch.Tensor | None = None) -> torch.Tensor:
    """``((residual or 0) + Transition(x)) * (mask or 1)``; x [..., C]."""
    check_inference(x, "transition")
    params = _parameters(module)
    key = cache_key(params, x, torch.bfloat16)
    blob = cached_blob(module, "_hip_transition_cache", key,
                       lambda: ops.transition_pack(*params, device=x.device))
    expansion = module.model_dim // module.linear_out.weight.shape[0]
    io = x if x.dtype in (torch.bfloat16, torch.float32) else x.float()
    res = ops.transition_forward(io, blob, expansion, eps=module.layernorm.eps, residual=residual,
                                 mask=mask, out=out)
    return res.to(x.dtype)


class SwiGLU(nn.Module):
    def __init__(self, channel_in: int, channel_out: int):
        super().__init__()
        self.linear = LinearNoBias(channel_in, channel_out * 2, init="relu")


class Transition(nn.Module):
    def __init__(self, channel: int, expansion_factor: int) -> None:
        super().__init__()
        self.model_dim = channel * expansion_factor
        self.layernorm = LayerNorm(channel)
        self.swiglu = SwiGLU(channel, self.model_dim)
        self.linear_out = LinearNoBias(self.model_dim, channel, init="final")

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return hip_transition(self, x)
