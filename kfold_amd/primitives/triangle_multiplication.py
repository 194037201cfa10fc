"""Triangle multiplicative update, ``kernel_backend="hip"``.

Drop-in for the reference's ``TriangleMultiplicationOutgoing/Incoming``
(src/kfold/model/primitives/triangle_multiplication.py:148,232): same constructor, same
parameter names, same ``forward(x, mask)``.  ``hip_triangular_mult`` is the function a
``kernel_backend == "hip"`` branch in the reference's ``forward`` would call, next to
``triton_triangluar_mult`` (:94-145), and follows that wrapper's conventions: inference
only, GPU tensors only, weights packed once and cached on the module, result in ``x.dtype``.
"""

from __future__ import annotations

import torch
from torch import nn

from .. import ops
from ._common import cache_key, cached_blob, check_inference
from .layers import LayerNorm, LinearNoBias


def _parameters(module: nn.Module):
    return (module.layernorm_in.weight, module.layernorm_in.bias, module.linear_p_in.weight,
            module.linear_g_in.weight, module.layernorm_out.weight, module.layernorm_out.bias,
            module.linear_p_out.weight, module.linear_g_out.weight)


@torch.compiler.disable
def hip_triangular_mult(module: nn.Module, x: torch.Tensor, mask: torch.Tensor,
                        direction: str) -> torch.Tensor:
    check_inference(x, "triangle multiplication")
    params = _parameters(module)
    # the kernels always compute in bf16 MFMA / fp32 accumulation, whatever autocast says
    key = cache_key(params, x, torch.bfloat16)
    blob = cached_blob(module, "_hip_multiplication_cache", key,
                       lambda: ops.trimul_pack(*params, device=x.device))
    io = x if x.dtype in (torch.bfloat16, torch.float32) else x.float()
    out = ops.trimul_forward(io, mask, blob, direction, eps=module.layernorm_in.eps)
    return out.to(x.dtype)


class _TriangleMultiplication(nn.Module):
    direction = ""

    def __init__(self, dim: int = 128, kernel_backend: str = "hip") -> None:
        super().__init__()
        if kernel_backend != "hip":
            raise ValueError(
                f"kfold_amd implements kernel_backend='hip' only, got {kernel_backend!r}; "
                "use the reference modules for the torch/triton/cuequiv backends")
        self.kernel_backend = kernel_backend
        self.layernorm_in = LayerNorm(dim)
        self.linear_p_in = LinearNoBias(dim, 2 * dim, init="default")
        self.linear_g_in = LinearNoBias(dim, 2 * dim, init="gating")
        self.layernorm_out = LayerNorm(dim)
        self.linear_p_out = LinearNoBias(dim, dim, init="final")
        self.linear_g_out = LinearNoBias(dim, dim, init="gating")

    def forward(self, x: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
        """x [B, N, N, D], mask [B, N, N] -> [B, N, N, D]."""
        return hip_triangular_mult(self, x, mask, direction=self.direction)


class TriangleMultiplicationOutgoing(_TriangleMultiplication):
    """Algorithm 12."""

    direction = "outgoing"


class TriangleMultiplicationIncoming(_TriangleMultiplication):
    """Algorithm 13."""

    direction = "incoming"
