"""Seeded synthetic inputs and random-init weights for tests and benchmarks.

Values are drawn in fp32 on the CPU from ``torch.Generator().manual_seed(seed)`` and cast or
moved afterwards, so a CPU run and a GPU run see the same numbers.  Weight rule: every
projection / gate matrix ~ trunc-normal(std 0.02, +-2 sigma); LayerNorm scale 1, offset 0;
linear biases 0 — drawn per parameter in ``named_parameters()`` order.
"""

from __future__ import annotations

import torch


@torch.no_grad()
def init_weights_(module: torch.nn.Module, seed: int = 0, std: float = 0.02) -> torch.nn.Module:
    gen = torch.Generator().manual_seed(seed)
    for name, p in module.named_parameters():
        if p.dim() >= 2:
            w = torch.empty(p.shape, dtype=torch.float32)
            torch.nn.init.trunc_normal_(w, mean=0.0, std=std, a=-2 * std, b=2 * std, generator=gen)
            p.copy_(w.to(p.dtype))
        elif name.endswith("bias"):
            p.zero_()
        else:                       # 1-D "weight": a LayerNorm scale
            p.fill_(1.0)
    return module


def token_mask(n: int, n_pad: int) -> torch.Tensor:
    """[1, n] bool, the last ``n_pad`` tokens are padding."""
    m = torch.ones(1, n, dtype=torch.bool)
    if n_pad:
        m[:, n - n_pad:] = False
    return m


def pair_mask_from_tokens(tok: torch.Tensor) -> torch.Tensor:
    """pair_mask[b, i, j] = tok[b, i] & tok[b, j]  (reference: model/model.py:516)."""
    return tok[:, :, None] & tok[:, None, :]


def pair_inputs(n: int, c_z: int = 128, n_pad: int = 0, seed: int = 0):
    """z [1, n, n, c_z] fp32 ~ N(0,1), token mask [1, n], pair mask [1, n, n] (bool)."""
    gen = torch.Generator().manual_seed(seed)
    z = torch.randn(1, n, n, c_z, generator=gen, dtype=torch.float32)
    tok = token_mask(n, n_pad)
    return z, tok, pair_mask_from_tokens(tok)


def single_inputs(n: int, c_s: int = 384, seed: int = 1, samples: int | None = None):
    """s [1, n, c_s] (or [1, samples, n, c_s]) fp32 ~ N(0,1)."""
    gen = torch.Generator().manual_seed(seed)
    shape = (1, n, c_s) if samples is None else (1, samples, n, c_s)
    return torch.randn(*shape, generator=gen, dtype=torch.float32)


def n_pad_for(n: int, frac: float) -> int:
    return int(round(frac * n))
