"""HIP transition, pair-bias projection and pair-bias attention vs the fp32 oracle."""

import pytest
import torch

from kfold_amd import synthetic
from tests.util import assert_close

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _pair(ref_cls, hip_cls, args, seed=0, std=0.02, tweak=None):
    ref = ref_cls(*args).eval()
    synthetic.init_weights_(ref, seed, std=std)
    if tweak:
        tweak(ref)
    hip = hip_cls(*args).eval()
    hip.load_state_dict(ref.state_dict())
    return ref, hip.to(DEV)


def _affine(ref):
    g = torch.Generator().manual_seed(77)
    with torch.no_grad():
        for name, p in ref.named_parameters():
            if p.dim() == 1:
                if name.endswith("bias"):
                    p.copy_(0.1 * torch.randn(p.shape, generator=g))
                else:
                    p.copy_(1 + 0.2 * torch.randn(p.shape, generator=g))


@pytest.mark.parametrize("channel,expansion,rows", [(128, 2, 1000), (128, 4, 333), (384, 4, 70),
                                                     (768, 2, 33), (256, 4, 1000), (256, 2, 77)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_transition_parity(channel, expansion, rows, dtype):
    from kfold_amd.layers import Transition, hip_transition
    from oracle import torch_path as O

    print(f"case transition C={channel} E={expansion} rows={rows} {dtype}", flush=True)
    ref, hip = _pair(O.Transition, Transition, (channel, expansion), std=0.05, tweak=_affine)
    x = torch.randn(rows, channel, generator=torch.Generator().manual_seed(rows)).to(dtype)
    with torch.no_grad():
        want = ref(x.float())
        got = hip(x.to(DEV))
        assert got.dtype == dtype
        assert_close(got, want, "transition", auto_scale=True)
        # fused residual (in place) and, for the pair kernel, the row mask
        xin = x.to(DEV).clone()
        mask = (torch.rand(rows, generator=torch.Generator().manual_seed(1)) > 0.3)
        if channel in (128, 256):          # the fused pair-track kernels take the row mask
            hip_transition(hip, xin, residual=xin, mask=mask.to(DEV), out=xin)
            want2 = (x.float() + want) * mask[:, None]
            assert (xin.cpu()[~mask] == 0).all()
        else:
            hip_transition(hip, xin, residual=xin, out=xin)
            want2 = x.float() + want
        assert_close(xin, want2, "transition residual", rel_fro=5e-3, auto_scale=True)


@pytest.mark.parametrize("n", [40, 96, 130])
def test_pair_bias_projection_and_trunk_apb(n):
    """Config 4a shape family: bias from z, 16 heads x 24, token padding."""
    from kfold_amd import modules as M
    from oracle import torch_path as O

    print(f"case pair bias + apb n={n}", flush=True)
    ref = O.PairSingleBlock().eval()
    synthetic.init_weights_(ref, 5, std=0.05)
    _affine(ref)
    hip = M.PairSingleBlock().eval()
    hip.load_state_dict(ref.state_dict())
    hip.to(DEV)
    z, tok, pm = synthetic.pair_inputs(n, 128, synthetic.n_pad_for(n, 0.12), seed=n)
    s = synthetic.single_inputs(n, 384, seed=n + 1)
    zb, sb = z.bfloat16(), s.bfloat16()
    with torch.no_grad():
        bias = ref.linear_pair_bias(ref.layernorm_z(zb.float())).movedim(-1, -3)
        want = ref.attention(sb.float(), None, bias, tok.float())
        # module interface with a dense bias (drop-in for SelfAttentionPairBias.forward)
        got = hip.attention(sb.to(DEV), None, bias.to(DEV), tok.to(DEV))
        assert_close(got, want, "apb module, dense bias", auto_scale=True)
        # fused: bias tiles straight from z
        from kfold_amd import ops
        tiles_dense = ops.bias_tiles_from_dense(bias.to(DEV).contiguous())
        blob = ops.pair_bias_pack(ref.layernorm_z.weight, ref.layernorm_z.bias,
                                  ref.linear_pair_bias.weight, device=torch.device(DEV))
        tiles = ops.pair_bias_project(zb.to(DEV), blob, 16)
        nb = (n + 31) // 32
        # bf16 tiles [h][qb][kb][chunk c][lane = query + 32*half][j]: element j of chunk c is
        # accumulator register v = 8c + j, i.e. key 8*(v//4) + 4*half + v%4
        t1 = tiles.view(torch.bfloat16).view(16, nb, nb, 2, 2, 32, 8).float()
        t2 = tiles_dense.view(torch.bfloat16).view(16, nb, nb, 2, 2, 32, 8).float()
        ar = torch.arange
        v = 8 * ar(2)[:, None, None] + ar(8)[None, None, :]                              # [c, 1, j]
        key32 = 8 * (v // 4) + 4 * ar(2)[None, :, None] + v % 4                          # [c, half, j]
        k = ar(nb)[:, None, None, None] * 32 + key32[None]                               # [kb, c, half, j]
        q = ar(nb)[:, None] * 32 + ar(32)[None, :]                                       # [qb, query]
        valid_q = (q < n)[None, :, None, None, None, :, None]
        valid_k = (k < n)[None, None, :, :, :, None, :]
        sel = (valid_q & valid_k).expand_as(t1).to(DEV)
        assert_close(t1[sel], t2[sel], "pair bias tiles", max_abs=3e-2, mean_abs=3e-3, rel_fro=1e-2)


def test_apb_functional_normalised_inputs_and_full_mask():
    from kfold_amd.layers import SelfAttentionPairBias, hip_attention_pair_bias
    from oracle import torch_path as O

    print("case apb functional", flush=True)
    ref, hip = _pair(O.SelfAttentionPairBias, SelfAttentionPairBias, (384, 16, None, "confidence"),
                     seed=3, std=0.05)
    with torch.no_grad():
        ref.linear_q.bias.copy_(0.2 * torch.randn(384, generator=torch.Generator().manual_seed(9)))
    hip.load_state_dict(ref.state_dict())
    L = 75
    g = torch.Generator().manual_seed(4)
    x = torch.randn(2, L, 384, generator=g)
    bias = torch.randn(2, 16, L, L, generator=g)
    mask = torch.rand(2, L, generator=g) > 0.25
    mask[1] = False                                   # one batch entry with every key masked
    with torch.no_grad():
        want = O.torch_attention_pair_bias(ref, x, x, bias, mask)
        xd = x.to(DEV)
        got = hip_attention_pair_bias(hip, xd, xd, bias.to(DEV), mask.to(DEV), call_site="confidence")
    assert_close(got, want, "apb functional (fp32 io, per-batch bias, fully masked batch)", auto_scale=True)


@pytest.mark.parametrize("s_shared", [False, True])
def test_apb_diffusion_variant(s_shared):
    """Config 4b shape family: 5 samples share one pair bias, c_a 768, 16 heads x 48, AdaLN."""
    from kfold_amd.layers import SelfAttentionPairBias
    from oracle import torch_path as O

    print(f"case apb diffusion s_shared={s_shared}", flush=True)
    ref, hip = _pair(O.SelfAttentionPairBias, SelfAttentionPairBias, (768, 16, 384, "diffusion_global"),
                     seed=6, std=0.03, tweak=_affine)
    L, S = 100, 5
    g = torch.Generator().manual_seed(8)
    a = torch.randn(1, S, L, 768, generator=g).bfloat16()
    s = torch.randn(1, 1 if s_shared else S, L, 384, generator=g).bfloat16()
    bias = torch.randn(1, 1, 16, L, L, generator=g)
    mask = torch.ones(1, 1, L, dtype=torch.bool)
    mask[..., L - 12:] = False
    with torch.no_grad():
        want = ref(a.float(), s.float().expand(1, S, L, 384), bias, mask)
        got = hip(a.to(DEV), s.to(DEV), bias.to(DEV), mask.to(DEV))
    assert got.shape == a.shape and got.dtype == a.dtype
    assert_close(got, want, "apb diffusion variant", auto_scale=True)


@pytest.mark.parametrize("cond", [False, True])
def test_cross_attention_local_windows(cond):
    """The atom transformer's attention: windows of 32 queries x 128 keys, c_atom 128, 4 heads x 32,
    one bias and key mask per window, 5 samples; with and without single conditioning."""
    from kfold_amd.layers import CrossAttentionPairBias
    from oracle import torch_path as O

    print(f"case cross attention windows cond={cond}", flush=True)
    cs = 128 if cond else None
    ref, hip = _pair(O.CrossAttentionPairBias, CrossAttentionPairBias, (128, 4, cs), seed=12, std=0.05,
                     tweak=_affine)
    S, W, Lq, Lk = 5, 23, 32, 128
    g = torch.Generator().manual_seed(14)
    aq = torch.randn(S, W, Lq, 128, generator=g).bfloat16()
    ak = torch.randn(S, W, Lk, 128, generator=g).bfloat16()
    sq = torch.randn(S, W, Lq, 128, generator=g).bfloat16() if cond else None
    sk = torch.randn(S, W, Lk, 128, generator=g).bfloat16() if cond else None
    bias = torch.randn(1, W, 4, Lq, Lk, generator=g)              # shared by the samples
    mask = torch.rand(1, W, Lk, generator=g) > 0.2
    mask[0, 3] = False                                            # a window with every key masked
    mask[0, 7, 40:] = False
    f = lambda t: None if t is None else t.float()
    with torch.no_grad():
        want = ref(aq.float(), ak.float(), f(sq), f(sk), bias, mask)
        d = lambda t: None if t is None else t.to(DEV)
        got = hip(aq.to(DEV), ak.to(DEV), d(sq), d(sk), bias.to(DEV), mask.to(DEV))
    assert got.shape == aq.shape and got.dtype == aq.dtype
    print(assert_close(got, want, "cross attention windows", auto_scale=True), flush=True)
    # odd window shape: 20 queries, 70 keys
    Lq2, Lk2 = 20, 70
    aq2, ak2 = aq[:1, :, :Lq2].contiguous(), ak[:1, :, :Lk2].contiguous()
    sq2 = None if sq is None else sq[:1, :, :Lq2].contiguous()
    sk2 = None if sk is None else sk[:1, :, :Lk2].contiguous()
    b2, m2 = bias[:, :, :, :Lq2, :Lk2].contiguous(), mask[:, :, :Lk2].contiguous()
    with torch.no_grad():
        want2 = ref(aq2.float(), ak2.float(), f(sq2), f(sk2), b2, m2)
        got2 = hip(aq2.to(DEV), ak2.to(DEV), d(sq2), d(sk2), b2.to(DEV), m2.to(DEV))
    assert_close(got2, want2, "cross attention, 20 x 70 windows", auto_scale=True)


# ---------------------------------------------------------------------------------------------
# fp32 arithmetic of the diffusion stack (reference: model/model.py:419 runs it outside autocast,
# kernels/triton/attention_pair_bias/dispatch.py:439,453 with fp32_dot_precision="ieee")
# ---------------------------------------------------------------------------------------------
F32_MAX_ABS = 1e-4          # against the fp32 oracle; bf16 arithmetic is at ~1e-2 on these inputs


@pytest.mark.parametrize("s_shared", [False, True])
def test_apb_diffusion_variant_fp32_arithmetic(s_shared):
    """Config 4b shape family with fp32 activations: 5 samples share one pair bias, c_a 768,
    16 heads x 48, AdaLN conditioning, 12 % of the keys padded — fp32-accurate on the bf16 matrix
    cores (three-way operand split)."""
    from kfold_amd.layers import SelfAttentionPairBias
    from oracle import torch_path as O

    print(f"case apb diffusion fp32 arithmetic s_shared={s_shared}", flush=True)
    ref, hip = _pair(O.SelfAttentionPairBias, SelfAttentionPairBias, (768, 16, 384, "diffusion_global"),
                     seed=6, std=0.03, tweak=_affine)
    L, S = 100, 5
    g = torch.Generator().manual_seed(8)
    a = torch.randn(1, S, L, 768, generator=g)
    s = torch.randn(1, 1 if s_shared else S, L, 384, generator=g)
    bias = torch.randn(1, 1, 16, L, L, generator=g)
    mask = torch.ones(1, 1, L, dtype=torch.bool)
    mask[..., L - 12:] = False
    with torch.no_grad():
        want = ref(a, s.expand(1, S, L, 384), bias, mask)
        got = hip(a.to(DEV), s.to(DEV), bias.to(DEV), mask.to(DEV))
        assert got.shape == a.shape and got.dtype == torch.float32
        e = assert_close(got, want, "apb diffusion variant, fp32 arithmetic", max_abs=F32_MAX_ABS, mean_abs=1e-5,
                         rel_fro=1e-5)
        print(e, flush=True)
        hip.arith = "bf16"                             # the same call in bf16 arithmetic, for scale
        got16 = hip(a.to(DEV), s.to(DEV), bias.to(DEV), mask.to(DEV))
    e16 = assert_close(got16, want, "apb diffusion variant, bf16 arithmetic on fp32 tensors", auto_scale=True)
    assert e["max_abs"] < 0.02 * e16["max_abs"], (e, e16)


@pytest.mark.parametrize("cond", [False, True])
def test_cross_attention_local_windows_fp32_arithmetic(cond):
    """32 x 128 windows (and an odd 20 x 70 shape) in fp32 arithmetic, a fully masked window and a
    partially masked one included."""
    from kfold_amd.layers import CrossAttentionPairBias
    from oracle import torch_path as O

    print(f"case cross attention windows fp32 arithmetic cond={cond}", flush=True)
    cs = 128 if cond else None
    ref, hip = _pair(O.CrossAttentionPairBias, CrossAttentionPairBias, (128, 4, cs), seed=12, std=0.05,
                     tweak=_affine)
    S, W, Lq, Lk = 2, 11, 32, 128
    g = torch.Generator().manual_seed(14)
    aq = torch.randn(S, W, Lq, 128, generator=g)
    ak = torch.randn(S, W, Lk, 128, generator=g)
    sq = torch.randn(S, W, Lq, 128, generator=g) if cond else None
    sk = torch.randn(S, W, Lk, 128, generator=g) if cond else None
    bias = torch.randn(1, W, 4, Lq, Lk, generator=g)
    mask = torch.rand(1, W, Lk, generator=g) > 0.2
    mask[0, 3] = False
    mask[0, 7, 40:] = False
    d = lambda t: None if t is None else t.to(DEV)
    with torch.no_grad():
        want = ref(aq, ak, sq, sk, bias, mask)
        got = hip(aq.to(DEV), ak.to(DEV), d(sq), d(sk), bias.to(DEV), mask.to(DEV))
    assert got.dtype == torch.float32
    print(assert_close(got, want, "cross attention windows, fp32 arithmetic", max_abs=F32_MAX_ABS, mean_abs=1e-5,
                       rel_fro=1e-5), flush=True)
    Lq2, Lk2 = 20, 70
    c = lambda t, n: None if t is None else t[:1, :, :n].contiguous()
    b2, m2 = bias[:, :, :, :Lq2, :Lk2].contiguous(), mask[:, :, :Lk2].contiguous()
    with torch.no_grad():
        want2 = ref(c(aq, Lq2), c(ak, Lk2), c(sq, Lq2), c(sk, Lk2), b2, m2)
        got2 = hip(d(c(aq, Lq2)), d(c(ak, Lk2)), d(c(sq, Lq2)), d(c(sk, Lk2)), b2.to(DEV), m2.to(DEV))
    assert_close(got2, want2, "cross attention, 20 x 70 windows, fp32 arithmetic", max_abs=F32_MAX_ABS,
                 mean_abs=1e-5, rel_fro=1e-5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_functional_entry_with_different_query_and_key_tensors(dtype):
    """``attention_pair_bias(module, x_q, x_k, ...)`` as CrossAttentionPairBias.forward calls it
    (layers/folding/attention_pair_bias.py:250-258): both sides already normalised, Lq != Lk."""
    from kfold_amd.layers import CrossAttentionPairBias, hip_attention_pair_bias
    from oracle import torch_path as O

    print(f"case functional entry, x_q != x_k, {dtype}", flush=True)
    ref, hip = _pair(O.CrossAttentionPairBias, CrossAttentionPairBias, (128, 4, None), seed=15, std=0.05)
    with torch.no_grad():
        ref.linear_q.bias.copy_(0.2 * torch.randn(128, generator=torch.Generator().manual_seed(9)))
    hip.load_state_dict(ref.state_dict())
    W, Lq, Lk = 9, 32, 128
    g = torch.Generator().manual_seed(16)
    xq = torch.randn(2, W, Lq, 128, generator=g).to(dtype)
    xk = torch.randn(2, W, Lk, 128, generator=g).to(dtype)
    bias = torch.randn(1, W, 4, Lq, Lk, generator=g)
    mask = torch.rand(1, W, Lk, generator=g) > 0.3
    with torch.no_grad():
        want = O.torch_attention_pair_bias(ref, xq.float(), xk.float(), bias, mask)
        got = hip_attention_pair_bias(hip, xq.to(DEV), xk.to(DEV), bias.to(DEV), mask.to(DEV),
                                      call_site="diffusion_local")
    assert got.shape == xq.shape and got.dtype == dtype
    if dtype == torch.float32:
        assert_close(got, want, "functional cross entry, fp32 arithmetic", max_abs=F32_MAX_ABS, mean_abs=1e-5,
                     rel_fro=1e-5)
    else:
        assert_close(got, want, "functional cross entry, bf16", auto_scale=True)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_prepared_pair_bias_gives_the_same_bits(dtype):
    """The sampler computes each block's pair bias once and uses it at every step
    (model/modules/ecsi.py:506-512): ``prepare_pair_bias`` converts it to tiles once; a call with the
    prepared bias equals the call with the dense one bit for bit, in both arithmetics."""
    from kfold_amd.layers import SelfAttentionPairBias, hip_attention_pair_bias, prepare_pair_bias

    print(f"case prepared pair bias {dtype}", flush=True)
    hip = SelfAttentionPairBias(768, 16, 384, "diffusion_global").eval()
    synthetic.init_weights_(hip, 6, std=0.03)
    hip.to(DEV)
    L, S = 70, 3
    g = torch.Generator().manual_seed(9)
    a = torch.randn(1, S, L, 768, generator=g).to(dtype).to(DEV)
    s = torch.randn(1, S, L, 384, generator=g).to(dtype).to(DEV)
    bias = torch.randn(1, 1, 16, L, L, generator=g).to(DEV)
    mask = (torch.rand(1, 1, L, generator=g) > 0.2).to(DEV)
    arith = "f32" if dtype == torch.float32 else "bf16"
    with torch.no_grad():
        want = hip(a, s, bias, mask)
        prepared = prepare_pair_bias(bias, arith)
        assert prepared.shape == bias.shape
        for _ in range(2):                                   # used again at the next step
            assert torch.equal(hip(a, s, prepared, mask), want)
        # one bias per sample
        bias_s = torch.randn(1, S, 16, L, L, generator=g).to(DEV)
        assert torch.equal(hip(a, s, prepare_pair_bias(bias_s, arith), mask), hip(a, s, bias_s, mask))
        # the functional entry takes it as well
        x = torch.randn(2, L, 768, generator=g).to(dtype).to(DEV)
        b2 = torch.randn(2, 16, L, L, generator=g).to(DEV)
        m2 = torch.ones(2, L, dtype=torch.bool).to(DEV)
        site = "diffusion_global"
        assert torch.equal(hip_attention_pair_bias(hip, x, x, prepare_pair_bias(b2, arith), m2, call_site=site),
                           hip_attention_pair_bias(hip, x, x, b2, m2, call_site=site))
        # prepared for the other arithmetic, or for another shape
        with pytest.raises(ValueError):
            hip(a, s, prepare_pair_bias(bias, "bf16" if arith == "f32" else "f32"), mask)
        with pytest.raises(ValueError):
            hip(a, s, prepare_pair_bias(bias[..., :L - 1, :L - 1].contiguous(), arith), mask)
        with pytest.raises(ValueError):
            hip(a, s, prepare_pair_bias(bias_s[:, :2].contiguous(), arith), mask)
