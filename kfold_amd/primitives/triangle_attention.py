"""Triangle attention around the starting / ending node, ``kernel_backend="hip"``.

Drop-in for the reference's ``TriangleAttentionStartingNode/EndingNode``
(src/kfold/model/primitives/triangle_attention.py:438,453): same constructor, parameter
names (``layer_norm``, ``linear``, ``mha.linear_{q,k,v,o,g}``) and ``forward(x, mask=None)``.
``hip_triangular_attn`` is what a ``kernel_backend == "hip"`` branch next to the triton one
(:404-408) would call; unlike the triton wrapper it takes the ``starting`` flag and reads
the ending node through strides, so the caller does not transpose (:400-402, :431-432).
"""

from __future__ import annotations

import torch
from torch import nn

from .. import ops
from ._common import cache_key, cached_blob, check_inf, check_inference
from .layers import LayerNorm, LinearNoBias


def _parameters(module: nn.Module):
    return (module.layer_norm.weight, module.layer_norm.bias, module.mha.linear_q.weight,
            module.mha.linear_k.weight, module.mha.linear_v.weight, module.mha.linear_g.weight,
            module.linear.weight, module.mha.linear_o.weight)


@torch.compiler.disable
def hip_triangular_attn(module: nn.Module, x: torch.Tensor, mask: torch.Tensor | None,
                        starting: bool) -> torch.Tensor:
    """x [*, I, J, C] and mask [*, I, J] in the caller's (untransposed) layout."""
    check_inference(x, "triangle attention")
    check_inf(module)
    params = _parameters(module)
    key = cache_key(params, x, torch.bfloat16)
    blob = cached_blob(module, "_hip_attention_cache", key,
                       lambda: ops.triattn_pack(*params, device=x.device))
    io = x if x.dtype in (torch.bfloat16, torch.float32) else x.float()
    out = ops.triattn_forward(io, mask, blob, module.no_heads, starting, eps=module.layer_norm.eps)
    return out.to(x.dtype)


class _AttentionWeights(nn.Module):
    """Parameter holder named like the reference's ``MultiHeadAttention`` (:172-244)."""

    def __init__(self, c_in: int, c_hidden: int, no_heads: int):
        super().__init__()
        self.linear_q = LinearNoBias(c_in, c_hidden * no_heads, init="default")
        self.linear_k = LinearNoBias(c_in, c_hidden * no_heads, init="default")
        self.linear_v = LinearNoBias(c_in, c_hidden * no_heads, init="default")
        self.linear_o = LinearNoBias(c_hidden * no_heads, c_in, init="final")
        self.linear_g = LinearNoBias(c_in, c_hidden * no_heads, init="gating")


class TriangleAttention(nn.Module):
    def __init__(self, c_in: int, no_heads: int, starting: bool, inf: float = 1e9,
                 kernel_backend: str = "hip") -> None:
        super().__init__()
        if kernel_backend != "hip":
            raise ValueError(
                f"kfold_amd implements kernel_backend='hip' only, got {kernel_backend!r}; "
                "use the reference modules for the torch/triton/cuequiv backends")
        assert c_in % no_heads == 0, f"c_in ({c_in}) must be divisible by no_heads ({no_heads})"
        self.c_in = c_in
        self.c_hidden = c_in // no_heads
        self.no_heads = no_heads
        self.starting = starting
        self.inf = inf
        self.kernel_backend = kernel_backend
        self.layer_norm = LayerNorm(c_in)
        self.linear = LinearNoBias(c_in, no_heads, init="default")
        self.mha = _AttentionWeights(c_in, self.c_hidden, no_heads)

    def forward(self, x: torch.Tensor, mask: torch.Tensor | None = None) -> torch.Tensor:
        """x [*, I, J, C_in], mask [*, I, J] (None = all valid) -> [*, I, J, C_in]."""
        return hip_triangular_attn(self, x, mask, self.starting)


class TriangleAttentionStartingNode(TriangleAttention):
    """Algorithm 14."""

    def __init__(self, c_in: int, no_heads: int, inf: float = 1e9, kernel_backend: str = "hip"):
        super().__init__(c_in, no_heads, starting=True, inf=inf, kernel_backend=kernel_backend)


class TriangleAttentionEndingNode(TriangleAttention):
    """Algorithm 15."""

    def __init__(self, c_in: int, no_heads: int, inf: float = 1e9, kernel_backend: str = "hip"):
        super().__init__(c_in, no_heads, starting=False, inf=inf, kernel_backend=kernel_backend)
