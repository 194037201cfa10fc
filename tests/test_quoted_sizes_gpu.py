"""Parity at the sizes the benchmark configurations are quoted on.

M   one block at N=768, bf16, 12 % token padding (the headline metric's shape)
C4a pair-bias attention, trunk variant, N=768 (bias projected from z [768,768,128])
C4b pair-bias attention, diffusion variant, N=768, 5 samples sharing one bias, 16 x 48
C3+ triangle attention at N=768 and N=1024 (LDS bias strip of 24 / 32 key blocks)
C2+ triangle multiplication at N=768
C5  48-block trunk at N=1024, bf16, 15 % padding

The oracle is evaluated in full where the host finishes in seconds (everything at N=768, one
block at N=1024) and on sampled rows otherwise; the 48-block run is checked through
size-independent properties per block plus oracle parity of its first and last block on the
stream values the HIP trunk itself produced.
"""

import time

import pytest
import torch

from kfold_amd import synthetic
from tests.test_block_gpu import check_stagewise
from tests.util import assert_close, assert_stream_close

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _trunk(num, seed=0, with_stream=False):
    from kfold_amd import modules as M
    from oracle import torch_path as O

    hip = M.PairformerTrunk(num).eval()
    synthetic.init_weights_(hip, seed)
    ref = O.PairSingleBlock(row_chunk=32).eval()
    ref.load_state_dict(hip.blocks[0].state_dict())
    stream = None
    if with_stream:
        stream = O.PairSingleBlock(row_chunk=32, stream_dtype=torch.bfloat16).eval()
        stream.load_state_dict(ref.state_dict())
    return ref, stream, hip.to(DEV)


def test_block_n768_metric_shape():
    """The headline shape: full oracle (fp32 and bf16-stream), every update on its own at the
    unscaled limits, masked positions exactly zero, bit determinism, padding invariance."""
    print("case block n=768", flush=True)
    n, n_pad = 768, synthetic.n_pad_for(768, 0.12)
    ref, stream, hip = _trunk(1, with_stream=True)
    z, tok, pm = synthetic.pair_inputs(n, 128, n_pad, seed=0)
    s = synthetic.single_inputs(n, 384, seed=1)
    zb, sb = z.bfloat16(), s.bfloat16()
    pmd, tokd = pm.to(DEV), tok.to(DEV)
    with torch.no_grad():
        t0 = time.time()
        zw, sw = ref(zb.float(), sb.float(), pm.float(), tok.float())
        zs, ss = stream(zb.float(), sb.float(), pm.float(), tok.float())
        print(f"  oracle x2 {time.time() - t0:.1f} s", flush=True)
        zg, sg = hip(zb.to(DEV), sb.to(DEV), pmd, tokd)
        print(assert_stream_close(zg, zs, zw, "block n=768 z"), flush=True)
        print(assert_stream_close(sg, ss, sw, "block n=768 s"), flush=True)
        assert (zg[~pmd] == 0).all()
        zg2, sg2 = hip(zb.to(DEV), sb.to(DEV), pmd, tokd)
        assert torch.equal(zg, zg2) and torch.equal(sg, sg2), "run-to-run results differ"
        # padding invariance: what padded tokens hold does not reach valid outputs
        nv = n - n_pad
        z2, s2 = zb.clone(), sb.clone()
        z2[:, nv:] = 50.0
        z2[:, :, nv:] = -50.0
        s2[:, nv:] = 30.0
        zg3, sg3 = hip(z2.to(DEV), s2.to(DEV), pmd, tokd)
        assert torch.equal(zg3[:, :nv, :nv], zg[:, :nv, :nv])
        assert torch.equal(sg3[:, :nv], sg[:, :nv])
    t0 = time.time()
    st = check_stagewise(ref, hip.blocks[0], zb.to(DEV), pm, "block n=768")
    print(f"  stagewise {time.time() - t0:.1f} s: " +
          ", ".join(f"{k} {v['max_abs']:.4f}/{v['mean_abs']:.5f}" for k, v in st.items()), flush=True)


@pytest.mark.parametrize("direction", ["outgoing", "incoming"])
def test_trimul_n768(direction):
    from kfold_amd import primitives as P
    from oracle import torch_path as O

    print(f"case trimul n=768 {direction}", flush=True)
    cls = "TriangleMultiplicationOutgoing" if direction == "outgoing" else "TriangleMultiplicationIncoming"
    ref = getattr(O, cls)(128).eval()
    synthetic.init_weights_(ref, 3)
    hip = getattr(P, cls)(128).eval()
    hip.load_state_dict(ref.state_dict())
    hip.to(DEV)
    z, _, pm = synthetic.pair_inputs(768, 128, synthetic.n_pad_for(768, 0.12), seed=2)
    zb = z.bfloat16()
    with torch.no_grad():
        want = ref(zb.float(), pm)
        got = hip(zb.to(DEV), pm.to(DEV))
    print(assert_close(got, want, f"trimul n=768 {direction}"), flush=True)
    assert (got.cpu()[~pm] == 0).all()


def _triattn_sampled(n, n_pad, starting, rows, seed):
    """HIP triangle attention on the whole tensor, the oracle on a sample of rows of x' (x for
    the starting node, x^T for the ending node): rows are independent given the pair bias, which
    is computed for the whole tensor."""
    from kfold_amd import primitives as P
    from oracle import torch_path as O

    cls = "TriangleAttentionStartingNode" if starting else "TriangleAttentionEndingNode"
    ref = getattr(O, cls)(128, 4).eval()
    synthetic.init_weights_(ref, seed)
    hip = getattr(P, cls)(128, 4).eval()
    hip.load_state_dict(ref.state_dict())
    hip.to(DEV)
    x, _, pm = synthetic.pair_inputs(n, 128, n_pad, seed=seed + 1)
    xb = x.bfloat16()
    with torch.no_grad():
        got = hip(xb.to(DEV), pm.to(DEV))
        got = (got if starting else got.transpose(1, 2))[0, rows].float().cpu()
        xt = xb.float() if starting else xb.float().transpose(1, 2)
        mt = pm.float() if starting else pm.float().transpose(1, 2)
        xn = ref.layer_norm(xt)
        bias = ref.linear(xn).movedim(-1, -3).unsqueeze(-4)
        mask5 = mt[..., :, None, None, :]
        want = ref.mha(xn[:, rows], xn[:, rows], bias, mask5[:, rows])[0]
    return got, want


@pytest.mark.parametrize("starting", [True, False])
@pytest.mark.parametrize("n,frac", [(768, 0.12), (1024, 0.15)])
def test_triattn_n768_n1024_sampled_rows(n, frac, starting):
    print(f"case triattn n={n} starting={starting}", flush=True)
    n_pad = synthetic.n_pad_for(n, frac)
    nv = n - n_pad
    rows = [0, 1, 31, 32, n // 2 + 3, nv - 1, nv, n - 1]     # valid rows and padded rows
    got, want = _triattn_sampled(n, n_pad, starting, rows, seed=40 + n)
    print(assert_close(got, want, f"triattn n={n} starting={starting}"), flush=True)


def test_apb_trunk_variant_n768():
    """Config 4a: s [1,768,384], 16 heads x 24, bias projected from z [1,768,768,128], 12 % padding."""
    from kfold_amd import modules as M
    from oracle import torch_path as O

    print("case C4a n=768", flush=True)
    n = 768
    ref = O.PairSingleBlock().eval()
    synthetic.init_weights_(ref, 5)
    hip = M.PairSingleBlock().eval()
    hip.load_state_dict(ref.state_dict())
    hip.to(DEV)
    z, tok, pm = synthetic.pair_inputs(n, 128, synthetic.n_pad_for(n, 0.12), seed=6)
    s = synthetic.single_inputs(n, 384, seed=7)
    zb, sb = z.bfloat16(), s.bfloat16()
    with torch.no_grad():
        bias = ref.linear_pair_bias(ref.layernorm_z(zb.float())).movedim(-1, -3)
        want = ref.attention(sb.float(), None, bias, tok.float())
        # fused path of the block: bias tiles straight from z, attention, no residual
        from kfold_amd import ops
        from kfold_amd.layers.attention_pair_bias import _parameters
        dev = torch.device(DEV)
        blob_pb = ops.pair_bias_pack(ref.layernorm_z.weight, ref.layernorm_z.bias,
                                     ref.linear_pair_bias.weight, device=dev)
        tiles = ops.pair_bias_project(zb.to(DEV), blob_pb, 16)
        att = hip.attention
        blob = ops.apb_pack(att.channel_a, att.num_heads, 0, device=dev, **_parameters(att))
        got = ops.apb_forward(sb.to(DEV), None, tiles, tok.to(DEV), blob, 16, 0, True, False)
        print(assert_close(got, want, "C4a fused (bias from z)"), flush=True)
        # module interface with the dense bias, as SelfAttentionPairBias.forward receives it
        got2 = att(sb.to(DEV), None, bias.to(DEV), tok.to(DEV))
        print(assert_close(got2, want, "C4a module (dense bias)"), flush=True)


@pytest.mark.parametrize("s_shared", [False, True])
def test_apb_diffusion_variant_n768(s_shared):
    """Config 4b: 5 samples share one pair bias, c_a 768, 16 heads x 48, AdaLN conditioning on
    s [.,768,384], N=768, 12 % padding, bf16."""
    from kfold_amd.layers import SelfAttentionPairBias
    from oracle import torch_path as O

    print(f"case C4b n=768 s_shared={s_shared}", flush=True)
    ref = O.SelfAttentionPairBias(768, 16, 384, "diffusion_global").eval()
    synthetic.init_weights_(ref, 8)
    hip = SelfAttentionPairBias(768, 16, 384, "diffusion_global").eval()
    hip.load_state_dict(ref.state_dict())
    hip.to(DEV)
    L, S = 768, 5
    g = torch.Generator().manual_seed(9)
    a = torch.randn(1, S, L, 768, generator=g).bfloat16()
    s = torch.randn(1, 1 if s_shared else S, L, 384, generator=g).bfloat16()
    bias = torch.randn(1, 1, 16, L, L, generator=g).bfloat16()
    mask = synthetic.token_mask(L, synthetic.n_pad_for(L, 0.12)).reshape(1, 1, L)
    with torch.no_grad():
        want = ref(a.float(), s.float().expand(1, S, L, 384), bias.float(), mask)
        got = hip(a.to(DEV), s.to(DEV), bias.to(DEV), mask.to(DEV))
    assert got.shape == a.shape and got.dtype == a.dtype
    print(assert_close(got, want, "C4b"), flush=True)


def test_trunk_48_blocks_n1024():
    """Config 5: 48 blocks, N=1024, bf16, 15 % trailing padding.  Per block: finite, masked
    positions exactly zero.  First block: every update against the oracle op on the same bf16
    input (unscaled limits).  Last block: every update against the oracle on the values the HIP
    trunk produced after 47 blocks, with an fp32 stream (|z| has grown past 8 there, where one
    bf16 step alone exceeds the limit).  Whole trunk: run-to-run bit determinism."""
    from oracle import torch_path as O

    print("case C5 48 x n=1024", flush=True)
    n, n_pad = 1024, synthetic.n_pad_for(1024, 0.15)
    ref, _, hip = _trunk(48)
    z, tok, pm = synthetic.pair_inputs(n, 128, n_pad, seed=0)
    s = synthetic.single_inputs(n, 384, seed=1)
    zb, sb = z.bfloat16(), s.bfloat16()
    pmd, tokd = pm.to(DEV), tok.to(DEV)

    t0 = time.time()
    st = check_stagewise(ref, hip.blocks[0], zb.to(DEV), pm, "C5 block 1")
    print(f"  block 1 stagewise {time.time() - t0:.1f} s: " +
          ", ".join(f"{k} {v['max_abs']:.4f}/{v['mean_abs']:.5f}" for k, v in st.items()), flush=True)

    def run(upto):
        zd, sd = zb.to(DEV), sb.to(DEV)
        with torch.no_grad():
            for i, blk in enumerate(hip.blocks[:upto]):
                zd, sd = blk(zd, sd, pmd, tokd, inplace_output=True)
                assert torch.isfinite(zd).all() and torch.isfinite(sd).all(), f"block {i}: not finite"
                assert (zd[~pmd] == 0).all(), f"block {i}: masked positions not zero"
        return zd, sd

    z47, s47 = run(47)
    with torch.no_grad():
        z48, s48 = hip.blocks[47](z47.clone(), s47.clone(), pmd, tokd, inplace_output=True)
        assert torch.isfinite(z48).all() and (z48[~pmd] == 0).all()
    zfull, sfull = run(48)
    assert torch.equal(zfull, z48) and torch.equal(sfull, s48), "run-to-run results differ"
    # the trunk module's own schedule (single tracks on a second stream) gives the same bits
    with torch.no_grad():
        zt, st_ = hip(zb.to(DEV), sb.to(DEV), pmd, tokd)
        torch.cuda.synchronize()
    assert torch.equal(zt, z48) and torch.equal(st_, s48), "two-stream trunk differs from the serial one"
    print(f"  after 48 blocks: |z| max {z48.abs().max().item():.2f} rms "
          f"{z48.float().pow(2).mean().sqrt().item():.3f}", flush=True)

    # last block on the trunk's own stream values, fp32 stream
    ref.load_state_dict(hip.blocks[47].state_dict())
    t0 = time.time()
    st = check_stagewise(ref, hip.blocks[47], z47.float(), pm, "C5 block 48 (fp32 stream)")
    print(f"  block 48 stagewise {time.time() - t0:.1f} s: " +
          ", ".join(f"{k} {v['max_abs']:.4f}/{v['mean_abs']:.5f}" for k, v in st.items()), flush=True)
    # single track of the last block: pair bias from z48, then the two in-place updates of s
    with torch.no_grad():
        zf = z48.float().cpu()
        bias = ref.linear_pair_bias(ref.layernorm_z(zf)).movedim(-1, -3)
        s_in = s47.float().cpu()
        s_mid = s_in + ref.attention(s_in, None, bias, tok.float())
        s_want = s_mid + ref.transition(s_mid)
        r_mid = s_mid.bfloat16().float()                  # the same with a bf16-rounded stream
        s_stream = (r_mid + ref.transition(r_mid)).bfloat16()
    print(assert_stream_close(s48, s_stream, s_want, "C5 block 48 single track"), flush=True)
