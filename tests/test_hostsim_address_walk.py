"""Every global access of the kernels stays inside its buffer at the quoted sizes and beyond.

The kernel sources run on the host execution model (``tests/hostsim``) at N = 768, 1024 and
1280 with every tensor they can touch — inputs, outputs, workspaces, packed weights, bias tiles —
allocated between inaccessible pages: an access outside a buffer ends the process with a report
naming the kernel, workgroup and thread.  To keep this a unit test only a sample of the workgroups
of each launch runs (the first and last ones, where the clamped and partial tiles are, and a
stride through the middle) and the MFMAs are skipped: the walk covers index arithmetic, grid
shapes and workspace carving, not numerics (``tests/test_hostsim_parity.py`` does those).
"""

from __future__ import annotations

import pytest
import torch

from kfold_amd import synthetic
from tests import hostsim

SIZES = [768, 1024, 1280]


def _pattern(shape, dtype=torch.bfloat16, seed=0):
    """Finite values without drawing hundreds of MB of normals: a random tile repeated."""
    g = torch.Generator().manual_seed(seed)
    n = 1
    for d in shape:
        n *= d
    tile = torch.randn(4099, generator=g)
    reps = (n + tile.numel() - 1) // tile.numel()
    return tile.repeat(reps)[:n].view(shape).to(dtype)


def _walk(stride, edge=24):
    return hostsim.host_backend(block_stride=stride, block_edge=edge, skip_math=True)


@pytest.mark.parametrize("n", SIZES)
def test_walk_pair_block(n):
    """Pairformer block, C = 128: tri-mul out/in, tri-attn start/end (strip kernel up to N = 1216,
    staged kernel above), pair transition, pair-bias projection, token-track attention + transition."""
    from kfold_amd import modules as M

    blk = M.PairSingleBlock().eval()
    synthetic.init_weights_(blk, 0)
    n_pad = synthetic.n_pad_for(n, 0.12)
    tok = synthetic.token_mask(n, n_pad)
    pm = synthetic.pair_mask_from_tokens(tok)
    with torch.no_grad(), _walk(stride=211) as arena:
        z = arena.like(_pattern((1, n, n, 128)))
        s = arena.like(_pattern((1, n, 384), seed=1))
        blk(z, s, arena.like(pm), arena.like(tok))
        launches = hostsim.load().hostsim_launch_count()
    assert launches > 0


@pytest.mark.parametrize("n,chunks", [(768, 3), (1000, 4), (1280, 3)])
def test_walk_pair_block_in_row_ranges(n, chunks):
    """The same block with every triangle op's core and output phase run over ranges of rows (offset
    pointers into planes, fragments, key codes, z): strip attention kernel at 768 and 1000 (N = 1000
    is no multiple of the 32-row blocks or the 128-row tiles), staged kernel at 1280."""
    from kfold_amd import modules as M

    blk = M.PairformerBlock(phase_row_chunks=chunks).eval()
    synthetic.init_weights_(blk, 0)
    tok = synthetic.token_mask(n, synthetic.n_pad_for(n, 0.12))
    pm = synthetic.pair_mask_from_tokens(tok)
    with torch.no_grad(), _walk(stride=211) as arena:
        z = arena.like(_pattern((1, n, n, 128)))
        before = hostsim.load().hostsim_launch_count()
        blk(z, arena.like(pm), inplace_output=True)
        # input phase + (core, output) per range for the four ops, and the transition
        assert hostsim.load().hostsim_launch_count() - before >= 4 * (1 + 2 * chunks) + 1


@pytest.mark.parametrize("n", [768, 1280])
def test_walk_triangular_block_c256(n):
    """Shipping trunk block: tri-mul at C = 256 (both directions) + transition x4."""
    from kfold_amd import modules as M

    blk = M.TriangularBlock(256).eval()
    synthetic.init_weights_(blk, 0)
    tok = synthetic.token_mask(n, synthetic.n_pad_for(n, 0.12))
    pm = synthetic.pair_mask_from_tokens(tok)
    with torch.no_grad(), _walk(stride=211) as arena:
        z = arena.like(_pattern((1, n, n, 256)))
        blk(z, arena.like(pm))


@pytest.mark.parametrize("n,batch", [(768, 1), (384, 4)])
def test_walk_triattn_c64_templates(n, batch):
    """Template-stack triangle attention: C = 64, 4 heads x 16, a batch of templates."""
    from kfold_amd import primitives as P

    tok = synthetic.token_mask(n, synthetic.n_pad_for(n, 0.1))
    pm = synthetic.pair_mask_from_tokens(tok).expand(batch, n, n).contiguous()
    for cls in (P.TriangleAttentionStartingNode, P.TriangleAttentionEndingNode):
        mod = cls(64, 4).eval()
        synthetic.init_weights_(mod, 1)
        with torch.no_grad(), _walk(stride=97) as arena:
            x = arena.like(_pattern((batch, n, n, 64)))
            mod(x, arena.like(pm))


def test_walk_template_stack_block_c64():
    """The apo template stack's Pairformer block: c = 64 (tri-mul and transition through the paths
    assembled from the token-track kernels), 4 templates of 384 tokens."""
    from kfold_amd import modules as M

    n, batch = 384, 4
    blk = M.PairformerBlock(64, 4).eval()
    synthetic.init_weights_(blk, 4)
    tok = synthetic.token_mask(n, synthetic.n_pad_for(n, 0.1))
    pm = synthetic.pair_mask_from_tokens(tok).expand(batch, n, n).contiguous()
    with torch.no_grad(), _walk(stride=307) as arena:
        z = arena.like(_pattern((batch, n, n, 64)))
        blk(z, arena.like(pm), inplace_output=True)


def test_walk_diffusion_attention_and_windows():
    """Diffusion-transformer pair-bias attention (5 samples, one bias, 768 tokens, 16 x 48) and
    the local cross-attention windows (32 queries x 128 keys)."""
    from kfold_amd.layers import attention_pair_bias as A

    n, S = 768, 5
    apb = A.SelfAttentionPairBias(768, 16, channel_s=384, call_site="diffusion_global").eval()
    synthetic.init_weights_(apb, 2)
    tok = synthetic.token_mask(n, synthetic.n_pad_for(n, 0.12))
    with torch.no_grad(), _walk(stride=53) as arena:
        a = arena.like(_pattern((1, S, n, 768)))
        s = arena.like(_pattern((1, S, n, 384), seed=3))
        bias = arena.like(_pattern((1, 1, 16, n, n), seed=4))
        apb(a, s, bias, arena.like(tok[:, None, :]))
    W = 40
    cross = A.CrossAttentionPairBias(128, 4, channel_s=128).eval()
    synthetic.init_weights_(cross, 3)
    with torch.no_grad(), _walk(stride=7) as arena:
        a_q = arena.like(_pattern((1, W, 32, 128)))
        a_k = arena.like(_pattern((1, W, 128, 128), seed=5))
        s_q = arena.like(_pattern((1, W, 32, 128), seed=6))
        s_k = arena.like(_pattern((1, W, 128, 128), seed=7))
        bias = arena.like(_pattern((1, W, 4, 32, 128), seed=8))
        mask = arena.like(torch.ones(1, W, 128, dtype=torch.bool))
        cross(a_q, a_k, s_q, s_k, bias, mask)


@pytest.mark.parametrize("c", [128, 256])
def test_walk_parcae_step(c):
    from kfold_amd import modules as M

    n = 1024
    step = M.ParcaeStep(c).eval()
    with torch.no_grad(), _walk(stride=101) as arena:
        z = arena.like(_pattern((1, n, n, c)))
        u = arena.like(_pattern((1, n, n, c), seed=9))
        step(z, u)


_TEETH = r"""
import sys, torch
sys.path.insert(0, {root!r})
from tests import hostsim
from kfold_amd import ops, primitives as P, synthetic
mod = P.TriangleMultiplicationOutgoing(128).eval()
synthetic.init_weights_(mod, 0)
n = 64
z, _, pm = synthetic.pair_inputs(n, 128, 0, seed=0)
with torch.no_grad(), hostsim.host_backend() as arena:
    zb = arena.like(z.bfloat16())
    mod(zb, pm)                                   # in bounds: passes
    print("in-bounds call ok", flush=True)
    short = arena.bytes(zb.numel() * 2 - 8192)    # 32 rows less than the kernel writes
    L = hostsim.load()
    need = L.kfh_trimul_workspace_bytes(n, 128)
    ws = arena.bytes(need)
    m8 = arena.like(pm.view(torch.uint8))
    rc = L.kfh_trimul_forward(zb.data_ptr(), m8.data_ptr(), mod._hip_multiplication_cache.data_ptr(), None,
                              short.data_ptr(), ws.data_ptr(), need, 1, n, 128, 0, 1e-5, 0, None)
print("not reached", rc)
"""


def test_the_walk_has_teeth():
    """An output buffer 8 KiB short of what the kernel writes: the run must die in
    trimul_out_kernel with the simulator's report (in a child process)."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, "-c", _TEETH.format(root=root)], capture_output=True, text=True,
                         timeout=300)
    assert "in-bounds call ok" in res.stdout
    assert "not reached" not in res.stdout and res.returncode != 0
    assert "[hostsim] invalid memory access" in res.stderr and "trimul_out_kernel" in res.stderr, res.stderr[-2000:]


def _untouched(arena, shape, dtype):
    """A guarded buffer that is never written (zero pages): at the sizes below the tensors are tens
    of GB of address space of which only the sampled workgroups' pages are ever touched."""
    n = 1
    for d in shape:
        n *= d
    return arena.bytes(n * torch.empty((), dtype=dtype).element_size(), 256).view(dtype).view(shape)


@pytest.mark.parametrize("what,n", [("pair_block", 3008), ("pair_block", 8192), ("wide_block", 6016),
                                    ("template_block", 4000), ("diffusion_attention", 8192)])
def test_walk_sizes_beyond_32_bit_offsets(what, n):
    """Element offsets pass 2^31 from N = 2897 on at C = 128 (N^2 * 2C) and every entry point takes
    N up to 8192: the first and last workgroups of every launch (and a stride between) at such sizes,
    where an index computed in 32 bits would leave its buffer."""
    from kfold_amd import layers, modules as M

    hs = hostsim.load()
    tok = synthetic.token_mask(n, synthetic.n_pad_for(n, 0.12))
    with torch.no_grad(), _walk(stride=16411) as arena:
        hs.hostsim_set_fill(0)
        try:
            if what == "pair_block":
                blk = synthetic.init_weights_(M.PairSingleBlock().eval(), 0)
                pm = synthetic.pair_mask_from_tokens(tok)
                blk(_untouched(arena, (1, n, n, 128), torch.bfloat16), _untouched(arena, (1, n, 384), torch.bfloat16),
                    arena.like(pm), arena.like(tok))
            elif what == "wide_block":
                blk = synthetic.init_weights_(M.TriangularBlock(256).eval(), 0)
                blk(_untouched(arena, (1, n, n, 256), torch.bfloat16), arena.like(synthetic.pair_mask_from_tokens(tok)))
            elif what == "template_block":
                blk = synthetic.init_weights_(M.PairformerBlock(64, 4).eval(), 0)
                pm = synthetic.pair_mask_from_tokens(tok).expand(2, n, n).contiguous()
                blk(_untouched(arena, (2, n, n, 64), torch.bfloat16), arena.like(pm), inplace_output=True)
            else:
                for dtype in (torch.float32, torch.bfloat16):
                    apb = synthetic.init_weights_(layers.SelfAttentionPairBias(768, 16, 384, "diffusion_global").eval(), 0)
                    apb(_untouched(arena, (1, 5, n, 768), dtype), _untouched(arena, (1, 5, n, 384), dtype),
                        _untouched(arena, (1, 1, 16, n, n), torch.float32), arena.like(tok.reshape(1, 1, n)))
        finally:
            hs.hostsim_set_fill(1)
