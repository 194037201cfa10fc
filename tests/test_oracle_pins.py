"""Pins for the oracle (``oracle/torch_path.py``).

The reference ships no tests, golden vectors or fixtures for this path, so the oracle is
pinned by (a) fp64 scalar-loop restatements of the index formulas on tiny sizes
(``oracle/brute.py``), (b) closed forms and special cases, (c) invariants of the math.  Each
check is chosen so that a plausible slip (swapped operand or index, wrong chunk half, dropped
bias or mask term, gate taken from the wrong tensor) breaks it.
"""

import math

import numpy as np
import pytest
import torch

from oracle import brute
from oracle import torch_path as O


def _rand_init(module, seed, std=0.4):
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for name, p in module.named_parameters():
            if p.dim() >= 2:
                p.copy_(std * torch.randn(p.shape, generator=g))
            elif name.endswith("bias"):
                p.copy_(0.3 * torch.randn(p.shape, generator=g))
            else:
                p.copy_(1 + 0.3 * torch.randn(p.shape, generator=g))
    return module.double().eval()


def _np_params(module):
    return {k: v.detach().double().numpy() for k, v in module.state_dict().items()}


def _rand(shape, seed):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64)


# ----------------------------------------------------------------------------- leaf layers
def test_layernorm_closed_forms():
    ln = O.LayerNorm(4)
    with torch.no_grad():
        ln.weight.copy_(torch.tensor([1.0, 2.0, 3.0, 4.0]))
        ln.bias.copy_(torch.tensor([0.5, -0.5, 0.25, 0.0]))
    # constant row -> (x - mu) = 0 -> beta
    assert torch.allclose(ln(torch.full((2, 4), 7.0)), ln.bias.expand(2, 4), atol=1e-6)
    # [-1, 1, -1, 1]: mu 0, biased var 1 -> x / sqrt(1 + eps)
    x = torch.tensor([[-1.0, 1.0, -1.0, 1.0]])
    want = x / math.sqrt(1 + 1e-5) * ln.weight + ln.bias
    assert torch.allclose(ln(x), want, atol=1e-6)
    # biased (1/n) variance, not 1/(n-1): [0, 0, 0, 2] has mu .5, var .75
    x = torch.tensor([[0.0, 0.0, 0.0, 2.0]])
    want = (x - 0.5) / math.sqrt(0.75 + 1e-5) * ln.weight + ln.bias
    assert torch.allclose(ln(x), want, atol=1e-6)
    # statistics are taken in fp32 even for a bf16 input, result cast back
    xb = torch.randn(3, 4).bfloat16()
    assert ln(xb).dtype == torch.bfloat16


def test_transition_and_adaln_vs_brute():
    t = _rand_init(O.Transition(6, 2), 1)
    x = _rand((5, 6), 2)
    assert np.allclose(t(x).detach().numpy(), brute.transition(x.numpy(), _np_params(t)), atol=1e-10)
    a = _rand_init(O.AdaLN(6, 4), 3)
    av, sv = _rand((5, 6), 4), _rand((5, 4), 5)
    assert np.allclose(a(av, sv).detach().numpy(), brute.adaln(av.numpy(), sv.numpy(), _np_params(a)),
                       atol=1e-10)


# ----------------------------------------------------------------- triangle multiplication
@pytest.mark.parametrize("cls,direction", [(O.TriangleMultiplicationOutgoing, "outgoing"),
                                            (O.TriangleMultiplicationIncoming, "incoming")])
def test_trimul_vs_brute(cls, direction):
    m = _rand_init(cls(4), 10)
    n = 5
    z = _rand((1, n, n, 4), 11)
    mask = (torch.rand(1, n, n, generator=torch.Generator().manual_seed(12)) > 0.3)
    got = m(z, mask.double())[0].detach().numpy()
    want = brute.tri_mul(z[0].numpy(), mask[0].numpy(), _np_params(m), direction)
    assert np.allclose(got, want, atol=1e-9), np.abs(got - want).max()


def test_trimul_zero_gate_weights_give_half_gates():
    m = _rand_init(O.TriangleMultiplicationOutgoing(4), 13)
    with torch.no_grad():
        m.linear_g_in.weight.zero_()
        m.linear_g_out.weight.zero_()
    z = _rand((1, 3, 3, 4), 14)
    ones = torch.ones(1, 3, 3, dtype=torch.float64)
    xn = m.layernorm_in(z)
    p = 0.5 * m.linear_p_in(xn)                      # sigmoid(0) = 1/2
    a, b = p[..., :4], p[..., 4:]
    y = torch.stack([torch.stack([(a[0, i] * b[0, j]).sum(0) for j in range(3)]) for i in range(3)])
    want = 0.5 * m.linear_p_out(m.layernorm_out(y))
    assert torch.allclose(m(z, ones)[0], want, atol=1e-10)


def test_trimul_incoming_is_outgoing_on_transpose_when_output_gate_is_flat():
    mo = _rand_init(O.TriangleMultiplicationOutgoing(4), 15)
    mi = O.TriangleMultiplicationIncoming(4).double().eval()
    with torch.no_grad():
        mo.linear_g_out.weight.zero_()
    mi.load_state_dict(mo.state_dict())
    z = _rand((1, 4, 4, 4), 16)
    mask = (torch.rand(1, 4, 4, generator=torch.Generator().manual_seed(17)) > 0.3).double()
    assert torch.allclose(mi(z, mask), mo(z.transpose(1, 2), mask.transpose(1, 2)), atol=1e-10)


# ---------------------------------------------------------------------- triangle attention
@pytest.mark.parametrize("starting", [True, False])
def test_triattn_vs_brute(starting):
    cls = O.TriangleAttentionStartingNode if starting else O.TriangleAttentionEndingNode
    m = _rand_init(cls(4, 2), 20)
    n = 4
    x = _rand((1, n, n, 4), 21)
    mask = (torch.rand(1, n, n, generator=torch.Generator().manual_seed(22)) > 0.3)
    mask[0, 2, :] = False                             # one fully masked row: stays finite
    got = m(x, mask.double())[0].detach().numpy()
    want = brute.tri_attn(x[0].numpy(), mask[0].numpy(), _np_params(m), heads=2, starting=starting)
    assert np.isfinite(got).all()
    assert np.allclose(got, want, atol=1e-8), np.abs(got - want).max()


def test_triattn_ending_equals_transposed_starting_and_row_chunking():
    ms = _rand_init(O.TriangleAttentionStartingNode(4, 2), 23)
    me = O.TriangleAttentionEndingNode(4, 2, row_chunk=2).double().eval()
    me.load_state_dict(ms.state_dict())
    x = _rand((1, 5, 5, 4), 24)
    mask = (torch.rand(1, 5, 5, generator=torch.Generator().manual_seed(25)) > 0.3).double()
    want = ms(x.transpose(1, 2), mask.transpose(1, 2)).transpose(1, 2)
    assert torch.allclose(me(x, mask), want, atol=1e-10)
    assert torch.allclose(me(x, None), ms(x.transpose(1, 2), None).transpose(1, 2), atol=1e-10)


def test_triattn_uniform_attention_and_single_key():
    m = _rand_init(O.TriangleAttentionStartingNode(4, 2), 26)
    with torch.no_grad():
        m.mha.linear_q.weight.zero_()                 # no q.k term
        m.linear.weight.zero_()                       # no pair bias
    x = _rand((1, 3, 3, 4), 27)
    xn = m.layer_norm(x)
    v = m.mha.linear_v(xn)                            # [1, I, K, C]
    g = torch.sigmoid(m.mha.linear_g(xn))
    # all keys valid: every query of row i gets mean_k v[i, k]
    want = m.mha.linear_o(g * v.mean(dim=2, keepdim=True))
    assert torch.allclose(m(x, torch.ones(1, 3, 3, dtype=torch.float64)), want, atol=1e-10)
    # only key 1 valid: every query of row i gets v[i, 1]
    mask = torch.zeros(1, 3, 3, dtype=torch.float64)
    mask[:, :, 1] = 1
    want = m.mha.linear_o(g * v[:, :, 1:2])
    assert torch.allclose(m(x, mask), want, atol=1e-10)


# --------------------------------------------------------------------- pair-bias attention
def test_apb_vs_brute_and_sample_sharing():
    m = _rand_init(O.SelfAttentionPairBias(6, 2, None), 30)
    L = 5
    a = _rand((1, L, 6), 31)
    bias = _rand((1, 2, L, L), 32)
    mask = torch.tensor([[1, 1, 0, 1, 1]], dtype=torch.float64)
    got = m(a, None, bias, mask)[0].detach().numpy()
    an = m.layernorm_a(a)[0].detach().numpy()
    want = brute.attention_pair_bias(an, an, bias[0].numpy(), mask[0].numpy(), _np_params(m), heads=2)
    assert np.allclose(got, want, atol=1e-9), np.abs(got - want).max()
    # a bias with a broadcast sample axis equals one call per sample
    a2 = _rand((1, 3, L, 6), 33)
    out = m(a2, None, bias[:, None], mask[:, None])
    for s in range(3):
        assert torch.allclose(out[:, s], m(a2[:, s], None, bias, mask), atol=1e-10)


def test_apb_conditioned_wiring():
    m = _rand_init(O.SelfAttentionPairBias(6, 2, 4, call_site="diffusion_global"), 34)
    L = 4
    a, s = _rand((1, L, 6), 35), _rand((1, L, 4), 36)
    bias = _rand((1, 2, L, L), 37)
    mask = torch.ones(1, L, dtype=torch.float64)
    an = torch.from_numpy(brute.adaln(a[0].numpy(), s[0].numpy(),
                                      {k[len("adaln_a."):]: v for k, v in _np_params(m).items()
                                       if k.startswith("adaln_a.")}))
    core = brute.attention_pair_bias(an.numpy(), an.numpy(), bias[0].numpy(), mask[0].numpy(),
                                     _np_params(m), heads=2)
    gate = torch.sigmoid(m.linear_ada_out(s))[0].detach().numpy()
    assert np.allclose(m(a, s, bias, mask)[0].detach().numpy(), gate * core, atol=1e-9)


# ------------------------------------------------------------------------------ invariants
def test_token_permutation_equivariance_and_crop_invariance():
    blk = _rand_init(O.PairformerBlock(4, 2), 40, std=0.3)
    n, nv = 6, 4
    z = _rand((1, n, n, 4), 41)
    tok = torch.zeros(1, n, dtype=torch.bool)
    tok[:, :nv] = True
    pm = (tok[:, :, None] & tok[:, None, :]).double()
    out = blk(z.clone(), pm)
    # masked positions are exactly zero at block level
    assert (out[0][~pm[0].bool()] == 0).all()
    # cropping to the valid tokens gives the same values there
    crop = blk(z[:, :nv, :nv].clone(), pm[:, :nv, :nv])
    assert torch.allclose(out[:, :nv, :nv], crop, atol=1e-9)
    # garbage in padded tokens does not leak into valid positions
    z2 = z.clone()
    z2[:, nv:] = 100 * _rand((1, n - nv, n, 4), 42)
    z2[:, :, nv:] = 100 * _rand((1, n, n - nv, 4), 43)
    assert torch.allclose(blk(z2, pm)[:, :nv, :nv], crop, atol=1e-9)
    # permuting tokens permutes the output
    perm = torch.tensor([2, 0, 3, 1, 5, 4])
    zp = z[:, perm][:, :, perm]
    pmp = pm[:, perm][:, :, perm]
    assert torch.allclose(blk(zp.clone(), pmp), out[:, perm][:, :, perm], atol=1e-9)


def test_block_wiring_and_in_place_residuals():
    blk = _rand_init(O.PairSingleBlock(8, 4, 2, 2), 50, std=0.3)
    n = 4
    z, s = _rand((1, n, n, 4), 51), _rand((1, n, 8), 52)
    tok = torch.tensor([[True, True, True, False]])
    pm = (tok[:, :, None] & tok[:, None, :]).double()
    # recompose from the individually pinned pieces
    pb = blk.pair_block
    zz = z.clone()
    zz = zz + pb.tri_mul_out(zz, pm)
    zz = zz + pb.tri_mul_in(zz, pm)
    zz = zz + pb.tri_att_start(zz, pm)
    zz = zz + pb.tri_att_end(zz, pm)
    zz = zz + pb.transition_z(zz)
    zz = zz * pm[..., None]
    bias = blk.linear_pair_bias(blk.layernorm_z(zz)).permute(0, 3, 1, 2)
    ss = s + blk.attention(s, None, bias, tok.double())
    ss = ss + blk.transition(ss)
    z_in, s_in = z.clone(), s.clone()
    z_out, s_out = blk(z_in, s_in, pm, tok.double())
    assert torch.allclose(z_out, zz, atol=1e-10) and torch.allclose(s_out, ss, atol=1e-10)
    # eval-mode adds mutate the caller's tensors (the final mask multiply does not)
    assert not torch.equal(z_in, z) and torch.equal(s_in, s_out)


# ------------------------------------------------------------------------ Parcae recurrence
def test_parcae_step_vs_brute_and_closed_forms():
    m = O.ParcaeStep(6)
    g = torch.Generator().manual_seed(31)
    with torch.no_grad():
        m.parcae_log_a.copy_(0.5 * torch.randn(6, generator=g))
        m.parcae_log_delta.copy_(torch.randn(6, generator=g))
        m.parcae_b_cont.copy_(torch.randn(6, 6, generator=g))          # not symmetric: [out, in] matters
        m.layernorm_z.weight.copy_(1 + 0.3 * torch.randn(6, generator=g))
        m.layernorm_z.bias.copy_(0.3 * torch.randn(6, generator=g))
    m = m.double().eval()
    z, u = _rand((5, 6), 32), _rand((5, 6), 33)
    got = m(z, u).detach().numpy()
    want = brute.parcae_step(z.numpy(), u.numpy(), _np_params(m))
    assert np.allclose(got, want, atol=1e-10)
    # freshly constructed module: a = decay_init exactly, B = -log(decay_init) * I
    f = O.ParcaeStep(4, decay_init=0.8).double()
    a, b = f.dynamics()
    assert torch.allclose(a, torch.full((4,), 0.8, dtype=torch.float64), atol=1e-12)
    assert torch.allclose(b, -math.log(0.8) * torch.eye(4, dtype=torch.float64), atol=1e-12)
    # b_cont = 0: pure channel-wise decay; log_delta -> -inf side: delta -> 0, a -> 1, state kept
    with torch.no_grad():
        f.parcae_b_cont.zero_()
    zz, uu = _rand((3, 4), 34), _rand((3, 4), 35)
    assert torch.allclose(f(zz, uu), 0.8 * zz, atol=1e-12)
    with torch.no_grad():
        f.parcae_log_delta.fill_(-40.0)
    assert torch.allclose(f(zz, uu), zz, atol=1e-12)


def test_cross_apb_windows_vs_brute():
    """Lq != Lk, one bias and one key mask per window, each side with its own norm."""
    m = _rand_init(O.CrossAttentionPairBias(6, 2, None), 41)
    W, Lq, Lk = 3, 2, 5
    aq, ak = _rand((W, Lq, 6), 42), _rand((W, Lk, 6), 43)
    bias = _rand((W, 2, Lq, Lk), 44)
    mask = torch.rand(W, Lk, generator=torch.Generator().manual_seed(45)) > 0.3
    mask[:, 0] = True
    got = m(aq, ak, None, None, bias, mask).detach().numpy()
    p = _np_params(m)
    for w in range(W):
        qn = np.array([brute._ln(r, p["layernorm_a_q.weight"], p["layernorm_a_q.bias"]) for r in aq[w].numpy()])
        kn = np.array([brute._ln(r, p["layernorm_a_k.weight"], p["layernorm_a_k.bias"]) for r in ak[w].numpy()])
        want = brute.attention_pair_bias(qn, kn, bias[w].numpy(), mask[w].numpy(), p, heads=2)
        assert np.allclose(got[w], want, atol=1e-9)
    # conditioned wiring: AdaLN per side, sigmoid(linear_ada_out(s_q)) gate on the result
    c = _rand_init(O.CrossAttentionPairBias(6, 2, 4), 46)
    sq, sk = _rand((W, Lq, 4), 47), _rand((W, Lk, 4), 48)
    got = c(aq, ak, sq, sk, bias, mask)
    qn, kn = c.adaln_a_q(aq, sq), c.adaln_a_k(ak, sk)
    core = O.torch_attention_pair_bias(c, qn, kn, bias, mask)
    assert torch.allclose(got, torch.sigmoid(c.linear_ada_out(sq)) * core, atol=1e-12)
    pc = _np_params(c)
    want0 = brute.attention_pair_bias(qn[0].detach().numpy(), kn[0].detach().numpy(), bias[0].numpy(),
                                      mask[0].numpy(), pc, heads=2)
    assert np.allclose(core[0].detach().numpy(), want0, atol=1e-9)


# ------------------------------------------------------------- trunk-level composition
def _zero_linear_weights(module):
    """All projections to zero: every update of a triangular block is then exactly zero."""
    with torch.no_grad():
        for name, p in module.named_parameters():
            if p.dim() >= 2:
                p.zero_()


def test_triangular_block_and_stack_wiring():
    """tri-mul out, tri-mul in, transition x4 recomposed from the individually pinned pieces; in
    place, no triangle attention, no final mask (modules/tri_stack.py:138-150)."""
    c, n = 4, 5
    blk = _rand_init(O.TriangularBlock(c), 60, std=0.3)
    assert blk.transition_z.swiglu.linear.weight.shape == (2 * 4 * c, c)
    assert not hasattr(blk, "tri_att_start")
    z = _rand((1, n, n, c), 61)
    tok = torch.tensor([[True, True, True, True, False]])
    pm = (tok[:, :, None] & tok[:, None, :]).double()
    zz = z.clone()
    zz = zz + blk.tri_mul_out(zz, pm)
    zz = zz + blk.tri_mul_in(zz, pm)
    zz = zz + blk.transition_z(zz)
    z_in = z.clone()
    out = blk(z_in, pm)
    assert out is z_in and torch.allclose(out, zz, atol=1e-10)
    assert out[0, -1, -1].abs().max() > 1e-3, "masked positions are not zeroed by this block"
    # the order of the two directions matters, so a swap would show
    sw = z.clone()
    sw = sw + blk.tri_mul_in(sw, pm)
    sw = sw + blk.tri_mul_out(sw, pm)
    sw = sw + blk.transition_z(sw)
    assert not torch.allclose(sw, zz, atol=1e-6)
    stack = _rand_init(O.TrianglularStack(c, 3), 62, std=0.3)
    want = z.clone()
    for b in stack.blocks:
        want = b(want.clone(), pm)
    assert torch.allclose(stack(z.clone(), pm), want, atol=1e-10)


def test_recurrent_trunk_wiring_and_closed_form():
    """model/model.py:522-529: u = z_inputs + lm_stack(z_lm); z = a z + B LN(u); z = main_stack(z)."""
    c, n = 4, 3
    trunk = _rand_init(O.ParcaeTrunk(c, lm_blocks=1, main_blocks=2), 70, std=0.3)
    g = torch.Generator().manual_seed(71)
    with torch.no_grad():
        trunk.parcae_log_a.copy_(0.5 * torch.randn(c, generator=g))
        trunk.parcae_log_delta.copy_(torch.randn(c, generator=g))
    z0, z_inputs, z_lm = _rand((1, n, n, c), 72), _rand((1, n, n, c), 73), _rand((1, n, n, c), 74)
    pm = torch.ones(1, n, n, dtype=torch.float64)
    step = O.ParcaeStep(c).double()
    step.load_state_dict({k: v for k, v in trunk.state_dict().items() if "stack" not in k})
    z = z0.clone()
    for _ in range(2):
        u = z_inputs + trunk.lm_stack(z_lm.clone(), pm)
        z = step(z, u)
        z = trunk.main_stack(z, pm)
    lm_before = z_lm.clone()
    got = trunk(z0.clone(), z_inputs, z_lm, pm, num_recycles=1)
    assert torch.allclose(got, z, atol=1e-10)
    assert torch.equal(z_lm, lm_before), "the LM embedding is reused by every recycle and must not change"
    # stacks that add nothing: the recurrence has the closed form of a geometric series,
    # z_R = a^(R+1) z_0 + (1 + a + ... + a^R) B LN(z_inputs + z_lm)
    _zero_linear_weights(trunk.lm_stack)
    _zero_linear_weights(trunk.main_stack)
    a, b = trunk.dynamics()
    drive = torch.nn.functional.linear(trunk.layernorm_z(z_inputs + z_lm), b)
    R = 3
    want = a ** (R + 1) * z0 + sum(a ** r for r in range(R + 1)) * drive
    assert torch.allclose(trunk(z0.clone(), z_inputs, z_lm, pm, num_recycles=R), want, atol=1e-10)


def test_stream_rounding_mode_of_the_block_oracle():
    """``stream_dtype`` rounds the residual stream after every in-place add and nothing else."""
    x = torch.tensor([1.0, 1.0, 1.0, -3.0])
    O._stream_add_(x, torch.tensor([2.0 ** -9, 2.0 ** -8, 3 * 2.0 ** -8, 2.0 ** -7]), torch.bfloat16)
    # bf16 keeps 8 significant bits: below half a step -> down, ties -> even, 3 - 2^-7 is a tie at
    # step 2^-6 between 2.984375 (odd) and 3.0 (even)
    assert x.tolist() == [1.0, 1.0, 1.015625, -3.0]
    y = torch.tensor([1.0])
    O._stream_add_(y, torch.tensor([2.0 ** -9]), None)
    assert y.item() == 1.0 + 2.0 ** -9
    c, n = 4, 4
    plain = _rand_init(O.PairformerBlock(c, 2), 80, std=0.3).float()
    same = O.PairformerBlock(c, 2, stream_dtype=torch.float32)
    bf = O.PairformerBlock(c, 2, stream_dtype=torch.bfloat16)
    same.load_state_dict(plain.state_dict())
    bf.load_state_dict(plain.state_dict())
    z = _rand((1, n, n, c), 81).float()
    pm = torch.ones(1, n, n)
    want = plain(z.clone(), pm)
    assert torch.equal(same(z.clone(), pm), want)
    z_bf = z.clone()
    got = bf(z_bf, pm)
    assert torch.equal(z_bf.to(torch.bfloat16).float(), z_bf), "the stream holds bf16 values after the block"
    d = (got - want).abs().max().item()
    assert 0 < d < 0.1, "rounding moves the result, by roundings only"
    # a block that adds nothing returns the input rounded once
    _zero_linear_weights(bf)
    assert torch.equal(bf(z.clone(), pm), z.to(torch.bfloat16).float())


def test_rounded_operand_mode_of_triangle_attention():
    """The rounded-operand mode restates the attention with its scalings folded into weights and
    an exp2 softmax.  With a rounding that changes nothing (fp32 operands) it has to reproduce
    the pinned forward — a wrong fold (log2 e, 1/sqrt d), a transposed bias or a mask slip would
    show — for partially masked rows and both node types; with bf16 operands it has to stay
    close at small logits (where bf16 operands cost ~1e-3) and a fully masked row must come out
    as uniform attention."""
    for cls in (O.TriangleAttentionStartingNode, O.TriangleAttentionEndingNode):
        m = cls(16, 2, row_chunk=3).eval()
        g = torch.Generator().manual_seed(31)
        with torch.no_grad():
            for name, p in m.named_parameters():
                if p.dim() >= 2:
                    p.copy_(0.5 * torch.randn(p.shape, generator=g))
                else:
                    p.copy_(1 + 0.2 * torch.randn(p.shape, generator=g))
        x = torch.randn(1, 7, 7, 16, generator=g)
        mask = torch.rand(1, 7, 7, generator=g) > 0.3
        mask[0, :, 0] = True
        mask[0, 0, :] = True                 # every row / column keeps a valid key
        with torch.no_grad():
            want = m(x, mask.float())
            m.mha.operand_dtype = torch.float32
            same = m(x, mask.float())
            m.mha.operand_dtype = torch.bfloat16
            rounded = m(x, mask.float())
            m.mha.operand_dtype = None
        assert torch.allclose(same, want, atol=2e-5, rtol=1e-5), (same - want).abs().max()
        err = (rounded - want).abs().max().item()
        assert 1e-5 < err < 0.15, err         # it does round, and only rounds
    # fully masked row -> uniform attention over all keys
    m = O.TriangleAttentionStartingNode(16, 2).eval()
    _ = [torch.nn.init.normal_(p, std=0.3) for p in m.parameters() if p.dim() >= 2]
    x = torch.randn(1, 5, 5, 16, generator=torch.Generator().manual_seed(3))
    mask = torch.ones(1, 5, 5)
    mask[0, 2, :] = 0
    with torch.no_grad():
        m.mha.operand_dtype = torch.float32
        got = m(x, mask)[0, 2]
        xn = m.layer_norm(x)[0, 2]
        v_mean = m.mha.linear_v(xn).mean(dim=0, keepdim=True)
        uniform = m.mha.linear_o(torch.sigmoid(m.mha.linear_g(xn)) * v_mean)
    assert torch.allclose(got, uniform, atol=1e-5)
