"""Writes tests/golden/host_model_vectors.pt: inputs and the outputs that the kernels' host build
(tests/hostsim) gives for them, for a few small cases of every operator family.

Run on the CPU:  python -m tests.golden.make_host_model_vectors
The GPU test tests/test_zy_host_model_vectors_gpu.py runs the same calls on the GPU and reports how far
the hardware's results are from the host build's (both round to bf16 in the same places, so nearly
all values should agree bit for bit): the link between what the host build verifies and what the
GPU executes.  Nothing here comes from the reference; the vectors are this library's own results.
"""

from __future__ import annotations

from pathlib import Path

import torch

from kfold_amd import synthetic

OUT = Path(__file__).resolve().parent / "host_model_vectors.pt"


def cases():
    """name -> (builder of the module, dict of CPU input tensors, call).  Shared by the generator
    and the GPU test so that both make the same calls."""
    from kfold_amd import layers, modules as M, primitives as P

    g = torch.Generator().manual_seed(1234)
    n = 24
    z, tok, pm = synthetic.pair_inputs(n, 128, 3, seed=5)
    zb = z.bfloat16()
    out = {}
    out["trimul_out_c128"] = (lambda: synthetic.init_weights_(P.TriangleMultiplicationOutgoing(128).eval(), 1, std=0.05),
                              {"x": zb, "mask": pm}, lambda m, t: m(t["x"], t["mask"]))
    out["trimul_in_c128"] = (lambda: synthetic.init_weights_(P.TriangleMultiplicationIncoming(128).eval(), 2, std=0.05),
                             {"x": zb, "mask": pm}, lambda m, t: m(t["x"], t["mask"]))
    out["triattn_start_c128"] = (lambda: synthetic.init_weights_(P.TriangleAttentionStartingNode(128, 4).eval(), 3, std=0.08),
                                 {"x": zb, "mask": pm}, lambda m, t: m(t["x"], t["mask"]))
    out["triattn_end_c128"] = (lambda: synthetic.init_weights_(P.TriangleAttentionEndingNode(128, 4).eval(), 4, std=0.08),
                               {"x": zb, "mask": pm}, lambda m, t: m(t["x"], t["mask"]))
    z256 = torch.randn(1, 20, 20, 256, generator=g).bfloat16()
    pm20 = synthetic.pair_mask_from_tokens(synthetic.token_mask(20, 2))
    out["trimul_out_c256"] = (lambda: synthetic.init_weights_(P.TriangleMultiplicationOutgoing(256).eval(), 5, std=0.03),
                              {"x": z256, "mask": pm20}, lambda m, t: m(t["x"], t["mask"]))
    z64 = torch.randn(2, 20, 20, 64, generator=g).bfloat16()
    pm64 = pm20.expand(2, 20, 20).contiguous()
    out["template_block_c64"] = (lambda: synthetic.init_weights_(M.PairformerBlock(64, 4).eval(), 6, std=0.05),
                                 {"x": z64, "mask": pm64}, lambda m, t: m(t["x"].clone(), t["mask"], inplace_output=True))
    x = torch.randn(300, 128, generator=g).bfloat16()
    out["transition_c128_e2"] = (lambda: synthetic.init_weights_(layers.Transition(128, 2).eval(), 7, std=0.05),
                                 {"x": x}, lambda m, t: m(t["x"]))
    x256 = torch.randn(200, 256, generator=g).bfloat16()
    out["transition_c256_e4"] = (lambda: synthetic.init_weights_(layers.Transition(256, 4).eval(), 8, std=0.05),
                                 {"x": x256}, lambda m, t: m(t["x"]))
    L, S = 40, 2
    for name, dtype in (("apb_diffusion_bf16", torch.bfloat16), ("apb_diffusion_f32", torch.float32)):
        a = torch.randn(1, S, L, 768, generator=g).to(dtype)
        s = torch.randn(1, S, L, 384, generator=g).to(dtype)
        bias = torch.randn(1, 1, 16, L, L, generator=g)
        mask = torch.ones(1, 1, L, dtype=torch.bool)
        mask[..., L - 5:] = False
        out[name] = (lambda: synthetic.init_weights_(layers.SelfAttentionPairBias(768, 16, 384, "diffusion_global").eval(), 9, std=0.03),
                     {"a": a, "s": s, "bias": bias, "mask": mask}, lambda m, t: m(t["a"], t["s"], t["bias"], t["mask"]))
    blk_z, blk_tok, blk_pm = synthetic.pair_inputs(24, 128, 3, seed=11)
    blk_s = synthetic.single_inputs(24, 384, seed=12)
    out["pair_single_block"] = (lambda: synthetic.init_weights_(M.PairSingleBlock().eval(), 10),
                                {"z": blk_z.bfloat16(), "s": blk_s.bfloat16(), "pm": blk_pm, "tok": blk_tok},
                                lambda m, t: m(t["z"].clone(), t["s"].clone(), t["pm"], t["tok"])[0])
    return out


def main() -> None:
    from tests import hostsim

    dev = hostsim.HostDevice("cpu")
    store = {}
    with torch.no_grad(), hostsim.host_backend():
        for name, (build, inputs, call) in cases().items():
            mod = build().to(dev)
            got = call(mod, {k: v.to(dev) for k, v in inputs.items()})
            store[name] = got.detach().clone().contiguous()
            print(name, tuple(got.shape), got.dtype, flush=True)
    torch.save(store, OUT)
    print(OUT, OUT.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
