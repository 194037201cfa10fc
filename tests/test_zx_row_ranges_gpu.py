"""Core and output phase of the triangle ops over ranges of result rows, the output phase of a range
on a second stream beside the core phase of the next, against the ops in one piece (bit-identical)."""

import pytest
import torch

from kfold_amd import synthetic

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def test_phases_over_row_ranges_give_the_same_bits():
    """Contraction / attention and the output phase over ranges of rows (the output phase of one range
    on a second stream beside the core phase of the next): the kernels of the whole op on offset
    pointers, so every result is bit-identical to the op run in one piece — in place, both
    directions / nodes, bf16 and fp32 tensors, C = 128 and 256."""
    _check_row_ranges(260, ((128, torch.bfloat16),), (2, 5), (2, 3))
    _check_row_ranges(260, ((128, torch.float32), (256, torch.bfloat16)), (3,), (3,), both=False)


def test_phases_over_row_ranges_at_the_benchmark_size():
    """N = 768: three ranges of 256 rows for the contraction (its 256-row tiles), four of 192 for the
    attention."""
    _check_row_ranges(768, ((128, torch.bfloat16),), (3,), (4,))


def _check_row_ranges(n, widths, trimul_chunks, triattn_chunks, both=True):
    from kfold_amd import ops, primitives as P

    print(f"case phases over row ranges n={n}", flush=True)
    on_gpu = str(DEV).startswith("cuda")
    side = torch.cuda.Stream(DEV) if on_gpu else None          # the host build runs the ranges in order
    g = torch.Generator().manual_seed(n)
    pm = (torch.rand(1, n, n, generator=g) > 0.15).to(DEV)
    for c, dtype in widths:
        z = torch.randn(1, n, n, c, generator=g).to(dtype).to(DEV)
        for cls in ("TriangleMultiplicationOutgoing", "TriangleMultiplicationIncoming")[0 if both else 1:]:
            mod = synthetic.init_weights_(getattr(P, cls)(c).eval(), 3, std=0.05).to(DEV)
            with torch.no_grad():
                mod(z[:, :8, :8].contiguous(), pm[:, :8, :8].contiguous())      # packs the weights
                blob, d = mod._hip_multiplication_cache, mod.direction
                whole = z.clone()
                ops.trimul_forward(whole, pm, blob, d, residual=whole, out=whole)
                for chunks in trimul_chunks:
                    calls = []
                    parts = z.clone()
                    ops.trimul_forward(parts, pm, blob, d, residual=parts, out=parts, row_chunks=chunks, side=side,
                                       before_write=lambda: calls.append(1))
                    if on_gpu:
                        torch.cuda.synchronize()
                    assert calls == [1]
                    assert torch.equal(parts, whole), f"tri-mul {cls} C={c} {dtype} in {chunks} ranges"
        if c != 128:
            continue
        for cls in ("TriangleAttentionStartingNode", "TriangleAttentionEndingNode")[0 if both else 1:]:
            mod = synthetic.init_weights_(getattr(P, cls)(c, 4).eval(), 4, std=0.08).to(DEV)
            with torch.no_grad():
                mod(z[:, :8, :8].contiguous(), pm[:, :8, :8].contiguous())
                blob = mod._hip_attention_cache
                whole = z.clone()
                ops.triattn_forward(whole, pm, blob, 4, mod.starting, residual=whole, out=whole)
                for chunks in triattn_chunks:
                    parts = z.clone()
                    ops.triattn_forward(parts, pm, blob, 4, mod.starting, residual=parts, out=parts,
                                        row_chunks=chunks, side=side)
                    if on_gpu:
                        torch.cuda.synchronize()
                    assert torch.equal(parts, whole), f"tri-attn {cls} {dtype} in {chunks} ranges"
