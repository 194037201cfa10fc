"""Results do not depend on the order in which the host execution model resumes the lanes.

Between two rendezvous points the model runs the lanes of a workgroup one after another; a kernel
that is missing a barrier between wavefronts (a write to LDS or to global scratch that another
wavefront reads) gets whatever that order happens to produce.  Every kernel family is therefore run
under three orders — lanes ascending, descending, wavefronts rotating from pass to pass — and has to
give the same bits.  (A race between wavefronts that real hardware would expose shows here as a
difference; lock-step effects inside one wavefront are outside what the model can vary.)

A further run takes the workgroups of every launch in descending order (nothing orders the workgroups
of a launch on the GPU, so nothing may depend on it), and another starts every workgroup with all of its LDS overwritten by 0xFF bytes (NaN as bf16 and
fp32): a kernel that reads LDS it has not written itself (left over from the workgroup that ran on
the compute unit before) gives other bits, or NaN.
"""

from __future__ import annotations

import pytest
import torch

from kfold_amd import synthetic
from tests import hostsim


def _run_all(build, run):
    outs = []
    for mode, poison in ((0, 0), (1, 0), (2, 0), (3, 0), (0, 1)):
        mod = build()
        with torch.no_grad(), hostsim.host_backend():
            hostsim.load().hostsim_set_schedule(mode)
            hostsim.load().hostsim_set_poison_lds(poison)
            try:
                outs.append([t.clone() for t in run(mod)])
            finally:
                hostsim.load().hostsim_set_schedule(0)
                hostsim.load().hostsim_set_poison_lds(0)
    for other in outs[1:]:
        for a, b in zip(outs[0], other):
            assert torch.equal(a, b)
    assert all(torch.isfinite(t.float()).all() for t in outs[0])


def test_pair_single_block_c128():
    from kfold_amd import modules as M

    n = 72
    z, tok, pm = synthetic.pair_inputs(n, 128, 9, seed=0)
    s = synthetic.single_inputs(n, 384, seed=1)

    def build():
        return synthetic.init_weights_(M.PairSingleBlock().eval(), 0)

    _run_all(build, lambda m: m(z.bfloat16(), s.bfloat16(), pm, tok))


def test_triangular_block_c256_and_template_block_c64():
    from kfold_amd import modules as M

    n = 70
    z, _, pm = synthetic.pair_inputs(n, 256, 9, seed=2)
    _run_all(lambda: synthetic.init_weights_(M.TriangularBlock(256).eval(), 1), lambda m: [m(z.bfloat16(), pm)])
    z64 = torch.randn(2, 40, 40, 64, generator=torch.Generator().manual_seed(3))
    pm64 = synthetic.pair_mask_from_tokens(synthetic.token_mask(40, 5)).expand(2, 40, 40).contiguous()
    _run_all(lambda: synthetic.init_weights_(M.PairformerBlock(64, 4).eval(), 2),
             lambda m: [m(z64.bfloat16(), pm64, inplace_output=True)])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_diffusion_attention_and_windows(dtype):
    """bf16 arithmetic on bf16 tensors, fp32 arithmetic (split operands) on fp32 tensors."""
    from kfold_amd.layers import CrossAttentionPairBias, SelfAttentionPairBias

    g = torch.Generator().manual_seed(5)
    L, S = 70, 3
    a = torch.randn(1, S, L, 768, generator=g).to(dtype)
    s = torch.randn(1, S, L, 384, generator=g).to(dtype)
    bias = torch.randn(1, 1, 16, L, L, generator=g)
    mask = torch.ones(1, 1, L, dtype=torch.bool)
    mask[..., L - 9:] = False
    _run_all(lambda: synthetic.init_weights_(SelfAttentionPairBias(768, 16, 384, "diffusion_global").eval(), 3),
             lambda m: [m(a, s, bias, mask)])
    W = 5
    aq = torch.randn(2, W, 32, 128, generator=g).to(dtype)
    ak = torch.randn(2, W, 128, 128, generator=g).to(dtype)
    sq = torch.randn(2, W, 32, 128, generator=g).to(dtype)
    sk = torch.randn(2, W, 128, 128, generator=g).to(dtype)
    cb = torch.randn(1, W, 4, 32, 128, generator=g)
    cm = torch.rand(1, W, 128, generator=g) > 0.2
    _run_all(lambda: synthetic.init_weights_(CrossAttentionPairBias(128, 4, 128).eval(), 4),
             lambda m: [m(aq, ak, sq, sk, cb, cm)])
