"""fp32 torch restatement of the reference's *torch* backend for the hot path.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).

Every class keeps the reference's parameter names so that a ``state_dict`` moves
between the reference modules, these oracle modules and the product modules
unchanged.  Each ``forward`` cites the reference lines it follows; paths are
relative to the reference's ``src/kfold``.

How each function is pinned (no reference-held vectors exist for this path, the
reference ships no tests):

* ``layer_norm``/``linear``/softmax: library routines, checked against closed
  forms in ``tests/test_oracle_pins.py``;
* triangle multiplication, triangle attention, pair-bias attention: checked
  against fp64 pure-Python loop restatements of the index formulas
  (``oracle/brute.py``) on tiny sizes, plus closed forms (zero gate weights give
  a 0.5 gate, zero query weights give uniform attention, single valid key
  returns that key's value) and invariants (ending == transpose of starting on
  the transposed input, incoming == outgoing contraction on the transposed
  input, token-permutation equivariance, crop-vs-pad invariance);
* block wiring (residual order, in-place adds, final mask): checked by
  recomposing the block from the individually pinned pieces.
"""

from __future__ import annotations

import math

import torch
import torch.nn as nn
import torch.nn.functional as F


def _up(x: torch.Tensor) -> torch.Tensor:
    """The reference's ``.float()`` upcasts; fp64 (only used by this oracle's fp64 pin tests)
    is left alone instead of being rounded down to fp32."""
    return x.to(torch.promote_types(x.dtype, torch.float32))


# ---------------------------------------------------------------------------
# leaf layers
# ---------------------------------------------------------------------------
class LayerNorm(nn.Module):
    """model/primitives/normalization.py:22-91 — statistics in fp32, cast back."""

    def __init__(self, dim: int, create_scale: bool = True, create_offset: bool = True,
                 eps: float = 1e-5):
        super().__init__()
        self.normalized_shape = dim
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim)) if create_scale else None
        self.bias = nn.Parameter(torch.zeros(dim)) if create_offset else None

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        # the reference upcasts with ``x.float()``; fp64 inputs (used only by the fp64 pin
        # tests of this oracle) are kept in fp64 instead of being rounded down to fp32
        ct = torch.promote_types(x.dtype, torch.float32)
        w = None if self.weight is None else self.weight.to(ct)
        b = None if self.bias is None else self.bias.to(ct)
        y = F.layer_norm(x.to(ct), (self.normalized_shape,), w, b, self.eps)
        return y.to(x.dtype)


class Linear(nn.Module):
    """model/primitives/linear.py:22-107 — ``y = x W^T (+ b)``, ``W`` is [out, in]."""

    def __init__(self, c_in: int, c_out: int, bias: bool = True):
        super().__init__()
        self.weight = nn.Parameter(torch.zeros(c_out, c_in))
        if bias:
            self.bias = nn.Parameter(torch.zeros(c_out))
        else:
            self.register_parameter("bias", None)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return F.linear(x, self.weight, self.bias)


class LinearNoBias(Linear):
    """model/primitives/linear.py:110-126."""

    def __init__(self, c_in: int, c_out: int):
        super().__init__(c_in, c_out, bias=False)


class SwiGLU(nn.Module):
    """model/primitives/activation.py:20-29 — ``silu(first half) * second half``."""

    def __init__(self, c_in: int, c_out: int):
        super().__init__()
        self.linear = LinearNoBias(c_in, 2 * c_out)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        u, v = self.linear(x).chunk(2, dim=-1)
        return F.silu(u) * v


class Transition(nn.Module):
    """model/layers/folding/transition.py:20-68."""

    def __init__(self, channel: int, expansion_factor: int):
        super().__init__()
        self.model_dim = channel * expansion_factor
        self.layernorm = LayerNorm(channel)
        self.swiglu = SwiGLU(channel, self.model_dim)
        self.linear_out = LinearNoBias(self.model_dim, channel)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.linear_out(self.swiglu(self.layernorm(x)))


class AdaLN(nn.Module):
    """model/primitives/normalization.py:94-125."""

    def __init__(self, channel_a: int, channel_s: int):
        super().__init__()
        self.layernorm_a = LayerNorm(channel_a, create_scale=False, create_offset=False)
        self.layernorm_s = LayerNorm(channel_s, create_scale=True, create_offset=False)
        self.linear_g = Linear(channel_s, channel_a)
        self.linear_bias = LinearNoBias(channel_s, channel_a)

    def forward(self, a: torch.Tensor, s: torch.Tensor) -> torch.Tensor:
        a = self.layernorm_a(a)
        s = self.layernorm_s(s)
        return torch.sigmoid(self.linear_g(s)) * a + self.linear_bias(s)


# ---------------------------------------------------------------------------
# triangle multiplication
# ---------------------------------------------------------------------------
class _TriangleMultiplication(nn.Module):
    """model/primitives/triangle_multiplication.py:148-313 (torch branch)."""

    direction = ""

    def __init__(self, dim: int = 128, kernel_backend: str = "torch"):
        super().__init__()
        self.kernel_backend = kernel_backend
        self.layernorm_in = LayerNorm(dim)
        self.linear_p_in = LinearNoBias(dim, 2 * dim)
        self.linear_g_in = LinearNoBias(dim, 2 * dim)
        self.layernorm_out = LayerNorm(dim)
        self.linear_p_out = LinearNoBias(dim, dim)
        self.linear_g_out = LinearNoBias(dim, dim)

    def forward(self, x: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
        # :212-229 (outgoing) / :296-313 (incoming)
        xn = self.layernorm_in(x)
        ab = self.linear_p_in(xn) * torch.sigmoid(self.linear_g_in(xn))
        ab = ab * mask.unsqueeze(-1)
        a, b = torch.chunk(_up(ab), 2, dim=-1)
        if self.direction == "outgoing":
            y = torch.einsum("bikd,bjkd->bijd", a, b)      # :224
        else:
            y = torch.einsum("bkid,bkjd->bijd", a, b)      # :308
        return self.linear_p_out(self.layernorm_out(y)) * torch.sigmoid(self.linear_g_out(xn))


class TriangleMultiplicationOutgoing(_TriangleMultiplication):
    direction = "outgoing"


class TriangleMultiplicationIncoming(_TriangleMultiplication):
    direction = "incoming"


# ---------------------------------------------------------------------------
# triangle attention
# ---------------------------------------------------------------------------
class MultiHeadAttention(nn.Module):
    """model/primitives/triangle_attention.py:172-335 (torch branch)."""

    def __init__(self, c_q: int, c_k: int, c_v: int, c_hidden: int, no_heads: int,
                 gating: bool = True, inf: float = 1e9):
        super().__init__()
        self.c_hidden = c_hidden
        self.no_heads = no_heads
        self.inf = inf
        self.linear_q = LinearNoBias(c_q, c_hidden * no_heads)
        self.linear_k = LinearNoBias(c_k, c_hidden * no_heads)
        self.linear_v = LinearNoBias(c_v, c_hidden * no_heads)
        self.linear_o = LinearNoBias(c_hidden * no_heads, c_q)
        self.linear_g = LinearNoBias(c_q, c_hidden * no_heads) if gating else None

    def forward(self, q_x, kv_x, tri_bias, mask):
        if getattr(self, "operand_dtype", None) is not None:
            return self._forward_rounded_operands(q_x, kv_x, tri_bias, mask)
        h = self.no_heads
        # :246-267 — project, split heads, move heads in front of the sequence axis
        q = self.linear_q(q_x).unflatten(-1, (h, -1)).transpose(-2, -3)
        k = self.linear_k(kv_x).unflatten(-1, (h, -1)).transpose(-2, -3)
        v = self.linear_v(kv_x).unflatten(-1, (h, -1)).transpose(-2, -3)
        q = q / math.sqrt(self.c_hidden)
        # :328-330, :132-152 — logits = q k^T, then += mask bias, then += pair bias
        logits = torch.matmul(q, k.transpose(-1, -2))
        logits = logits + (-self.inf) * (~mask.bool()).to(q.dtype)
        logits = logits + tri_bias
        o = torch.matmul(torch.softmax(logits, dim=-1), v).transpose(-2, -3)
        # :269-283 — gate with sigmoid(linear_g(q_x)), merge heads, project
        if self.linear_g is not None:
            g = torch.sigmoid(self.linear_g(q_x)).unflatten(-1, (h, -1))
            o = o * g
        return self.linear_o(o.flatten(-2))


    # -- what a reduced-precision matrix unit sees ------------------------------------------
    # Same formulas, with every operand of a matrix product rounded to ``operand_dtype`` first
    # (inputs, weights, q, k, v, the pair bias, the probabilities, the gated output), products
    # and sums in fp32, softmax statistics in fp32 on unrounded exponentials.  Scalings are
    # folded where a fused kernel folds them: 1/sqrt(d) and log2(e) into the query weights and
    # log2(e) into the bias (``tri_bias`` arrives unscaled), so the softmax runs on exp2.  Used to
    # separate operand rounding from defects when logits are large: a kernel that computes in
    # this precision should match THIS to normal tolerances whatever the logit magnitude.
    def _forward_rounded_operands(self, q_x, kv_x, tri_bias, mask):
        dt = self.operand_dtype

        def rnd(t):
            return t.to(dt).to(torch.float32)

        h = self.no_heads
        log2e = 1.4426950408889634
        xq, xk = rnd(q_x), rnd(kv_x)
        wq = rnd(self.linear_q.weight * (log2e / math.sqrt(self.c_hidden)))
        q = rnd(F.linear(xq, wq)).unflatten(-1, (h, -1)).transpose(-2, -3)
        k = rnd(F.linear(xk, rnd(self.linear_k.weight))).unflatten(-1, (h, -1)).transpose(-2, -3)
        v = rnd(F.linear(xk, rnd(self.linear_v.weight))).unflatten(-1, (h, -1)).transpose(-2, -3)
        logits = torch.matmul(q, k.transpose(-1, -2)) + rnd(tri_bias * log2e)
        valid = mask.bool().expand_as(logits)
        # a row without any valid key attends uniformly (what the finite -inf of the reference
        # gives while |logits| < 32, triangle_attention.py:328)
        none_valid = ~valid.any(dim=-1, keepdim=True)
        logits = torch.where(none_valid, torch.zeros_like(logits),
                             logits.masked_fill(~valid, float("-inf")))
        e = torch.exp2(logits - logits.amax(dim=-1, keepdim=True))
        o = torch.matmul(rnd(e), v) / e.sum(dim=-1, keepdim=True)
        o = o.transpose(-2, -3)
        if self.linear_g is not None:
            g = torch.sigmoid(F.linear(xq, rnd(self.linear_g.weight))).unflatten(-1, (h, -1))
            o = o * g
        return F.linear(rnd(o.flatten(-2)), rnd(self.linear_o.weight))


class TriangleAttention(nn.Module):
    """model/primitives/triangle_attention.py:338-434 (torch branch).

    ``row_chunk`` bounds the [rows, H, N, N] logits held at once; rows are
    independent so the result does not depend on it.
    """

    def __init__(self, c_in: int, no_heads: int, starting: bool, inf: float = 1e9,
                 kernel_backend: str = "torch", row_chunk: int | None = None):
        super().__init__()
        assert c_in % no_heads == 0
        self.c_in = c_in
        self.c_hidden = c_in // no_heads
        self.no_heads = no_heads
        self.starting = starting
        self.inf = inf
        self.kernel_backend = kernel_backend
        self.row_chunk = row_chunk
        self.layer_norm = LayerNorm(c_in)
        self.linear = LinearNoBias(c_in, no_heads)
        # the reference does not forward ``inf`` to the inner attention (:366-373): it keeps 1e9
        self.mha = MultiHeadAttention(c_in, c_in, c_in, self.c_hidden, no_heads)

    def forward(self, x: torch.Tensor, mask: torch.Tensor | None = None) -> torch.Tensor:
        if mask is None:                                     # :394-398
            mask = x.new_ones(x.shape[:-1])
        if not self.starting:                                # :400-402
            x = x.transpose(-2, -3)
            mask = mask.transpose(-1, -2)
        x = self.layer_norm(x)                               # :411
        # :416-422 — bias [*, I, J, H] -> [*, 1, H, I, J]; here I plays "query", J "key"
        od = getattr(self.mha, "operand_dtype", None)
        if od is not None:      # rounded-operand mode (see MultiHeadAttention): the bias product too
            xr = x.to(od).to(torch.float32)
            bias = (F.linear(xr, (self.linear.weight * 1.4426950408889634).to(od).to(torch.float32))
                    / 1.4426950408889634).movedim(-1, -3).unsqueeze(-4)
        else:
            bias = self.linear(x).movedim(-1, -3).unsqueeze(-4)
        mask5 = mask[..., :, None, None, :]                  # :414  [*, I, 1, 1, J]
        n_rows = x.shape[-3]
        step = self.row_chunk or n_rows
        outs = []
        for r0 in range(0, n_rows, step):
            xs = x[..., r0:r0 + step, :, :]
            outs.append(self.mha(xs, xs, bias, mask5[..., r0:r0 + step, :, :, :]))
        out = torch.cat(outs, dim=-3)
        if not self.starting:                                # :431-432
            out = out.transpose(-2, -3)
        return out


class TriangleAttentionStartingNode(TriangleAttention):
    def __init__(self, c_in: int, no_heads: int, inf: float = 1e9,
                 kernel_backend: str = "torch", row_chunk: int | None = None):
        super().__init__(c_in, no_heads, True, inf, kernel_backend, row_chunk)


class TriangleAttentionEndingNode(TriangleAttention):
    def __init__(self, c_in: int, no_heads: int, inf: float = 1e9,
                 kernel_backend: str = "torch", row_chunk: int | None = None):
        super().__init__(c_in, no_heads, False, inf, kernel_backend, row_chunk)


# ---------------------------------------------------------------------------
# pair-bias attention
# ---------------------------------------------------------------------------
def torch_attention_pair_bias(module, x_q, x_k, pair_bias, mask):
    """model/primitives/attention.py:75-94 + :239-271 + :122-168 (``"torch"`` kernel)."""
    h, dh = module.num_heads, module.head_dim
    q = module.linear_q(x_q).unflatten(-1, (h, dh)).transpose(-2, -3)
    k = module.linear_k(x_k).unflatten(-1, (h, dh)).transpose(-2, -3)
    v = module.linear_v(x_k).unflatten(-1, (h, dh)).transpose(-2, -3)
    bias = pair_bias - module.inf * _up((~mask.bool()).to(pair_bias.dtype))[..., None, None, :]   # :255-257
    scale = 1.0 / math.sqrt(dh)
    logits = torch.einsum("...qc,...kc->...qk", _up(q) * scale, _up(k))          # :156
    logits = logits + _up(bias)
    attn = torch.softmax(logits, dim=-1).to(v.dtype)
    av = torch.einsum("...qk,...kc->...qc", attn, v)                              # :166
    av = av.transpose(-2, -3).reshape(x_q.shape)                                  # :267
    g = torch.sigmoid(F.linear(x_q, module.linear_g.weight, module.linear_g.bias))
    return F.linear(g * av, module.linear_out.weight, module.linear_out.bias)    # :269-270


class SelfAttentionPairBias(nn.Module):
    """model/layers/folding/attention_pair_bias.py:30-158."""

    def __init__(self, channel_a: int, num_heads: int, channel_s: int | None,
                 call_site: str = "confidence", inf: float = 1e9, kernel_backend: str = "torch"):
        super().__init__()
        assert channel_a % num_heads == 0
        if call_site not in {"diffusion_global", "confidence"}:
            raise ValueError(f"Unsupported self APB call site: {call_site!r}")
        self.channel_a = channel_a
        self.num_heads = num_heads
        self.head_dim = channel_a // num_heads
        self.inf = inf
        self.call_site = call_site
        self.kernel_backend = kernel_backend
        self.use_single_conditioning = channel_s is not None
        self.linear_q = Linear(channel_a, channel_a)
        self.linear_k = LinearNoBias(channel_a, channel_a)
        self.linear_v = LinearNoBias(channel_a, channel_a)
        self.linear_g = LinearNoBias(channel_a, channel_a)
        self.linear_out = LinearNoBias(channel_a, channel_a)
        if self.use_single_conditioning:
            self.adaln_a = AdaLN(channel_a, channel_s)
            self.linear_ada_out = Linear(channel_s, channel_a)
        else:
            self.layernorm_a = LayerNorm(channel_a)

    def forward(self, a, s, pair_bias, mask):
        if self.use_single_conditioning:
            a = self.adaln_a(a, s)
        else:
            assert s is None
            a = self.layernorm_a(a)
        a = torch_attention_pair_bias(self, a, a, pair_bias, mask)
        if self.use_single_conditioning:
            a = torch.sigmoid(self.linear_ada_out(s)) * a                         # :155-157
        return a


class CrossAttentionPairBias(nn.Module):
    """model/layers/folding/attention_pair_bias.py:161-260 — attention of Lq queries over Lk
    keys inside local windows (leading dims ..., W), each side with its own LayerNorm / AdaLN."""

    def __init__(self, channel_a: int, num_heads: int, channel_s: int | None, inf: float = 1e9,
                 kernel_backend: str = "torch"):
        super().__init__()
        assert channel_a % num_heads == 0
        self.channel_a = channel_a
        self.num_heads = num_heads
        self.head_dim = channel_a // num_heads
        self.inf = inf
        self.kernel_backend = kernel_backend
        self.use_single_conditioning = channel_s is not None
        self.linear_q = Linear(channel_a, channel_a)
        self.linear_k = LinearNoBias(channel_a, channel_a)
        self.linear_v = LinearNoBias(channel_a, channel_a)
        self.linear_g = LinearNoBias(channel_a, channel_a)
        self.linear_out = LinearNoBias(channel_a, channel_a)
        if self.use_single_conditioning:
            self.adaln_a_q = AdaLN(channel_a, channel_s)
            self.adaln_a_k = AdaLN(channel_a, channel_s)
            self.linear_ada_out = Linear(channel_s, channel_a)
        else:
            self.layernorm_a_q = LayerNorm(channel_a)
            self.layernorm_a_k = LayerNorm(channel_a)

    def forward(self, a_q, a_k, s_q, s_k, pair_bias, mask):
        if self.use_single_conditioning:                                          # :241-244
            a_q = self.adaln_a_q(a_q, s_q)
            a_k = self.adaln_a_k(a_k, s_k)
        else:                                                                     # :245-248
            assert s_q is None and s_k is None
            a_q = self.layernorm_a_q(a_q)
            a_k = self.layernorm_a_k(a_k)
        a_q = torch_attention_pair_bias(self, a_q, a_k, pair_bias, mask)          # :250-258
        if self.use_single_conditioning:                                          # :260-262
            a_q = torch.sigmoid(self.linear_ada_out(s_q)) * a_q
        return a_q


# ---------------------------------------------------------------------------
# blocks
# ---------------------------------------------------------------------------
def _stream_add_(x: torch.Tensor, update: torch.Tensor, stream_dtype) -> None:
    """``x += update`` in place (primitives/utils.py:47-48).  With ``stream_dtype`` set the sum is
    rounded to that dtype (and kept in the tensor's own dtype): the values a residual stream
    stored in ``stream_dtype`` holds after the add, as under the reference's bf16 autocast
    (inference/runner.py:565-571) where ``z`` itself is a bf16 tensor."""
    x.add_(update)
    if stream_dtype is not None:
        x.copy_(x.to(stream_dtype))


class PairformerBlock(nn.Module):
    """model/modules/apo_module.py:107-172, eval mode (dropout is the identity).

    ``stream_dtype``: round the residual stream to this dtype after every in-place add
    (None = the all-fp32 oracle).  The arithmetic of every op stays fp32 either way."""

    def __init__(self, channel_z: int = 128, num_tri_heads: int = 4,
                 row_chunk: int | None = None, stream_dtype: torch.dtype | None = None):
        super().__init__()
        self.stream_dtype = stream_dtype
        self.tri_mul_out = TriangleMultiplicationOutgoing(channel_z)
        self.tri_mul_in = TriangleMultiplicationIncoming(channel_z)
        self.tri_att_start = TriangleAttentionStartingNode(channel_z, num_tri_heads,
                                                           row_chunk=row_chunk)
        self.tri_att_end = TriangleAttentionEndingNode(channel_z, num_tri_heads,
                                                       row_chunk=row_chunk)
        self.transition_z = Transition(channel_z, expansion_factor=2)

    def forward(self, z: torch.Tensor, pair_mask: torch.Tensor) -> torch.Tensor:
        # in eval mode the adds mutate the caller's tensor (primitives/utils.py:47-48)
        sd = self.stream_dtype
        _stream_add_(z, self.tri_mul_out(z, pair_mask), sd)
        _stream_add_(z, self.tri_mul_in(z, pair_mask), sd)
        _stream_add_(z, self.tri_att_start(z, pair_mask), sd)
        _stream_add_(z, self.tri_att_end(z, pair_mask), sd)
        _stream_add_(z, self.transition_z(z), sd)
        return z * pair_mask[..., None]


class TriangularBlock(nn.Module):
    """model/modules/tri_stack.py:96-151, eval mode: tri-mul out, tri-mul in, transition x4,
    every update added in place (:138-150); no triangle attention and no final mask."""

    def __init__(self, channel_z: int = 128, stream_dtype: torch.dtype | None = None):
        super().__init__()
        self.stream_dtype = stream_dtype
        self.tri_mul_out = TriangleMultiplicationOutgoing(channel_z)
        self.tri_mul_in = TriangleMultiplicationIncoming(channel_z)
        self.transition_z = Transition(channel_z, expansion_factor=4)

    def forward(self, z: torch.Tensor, pair_mask: torch.Tensor) -> torch.Tensor:
        sd = self.stream_dtype
        _stream_add_(z, self.tri_mul_out(z, pair_mask), sd)
        _stream_add_(z, self.tri_mul_in(z, pair_mask), sd)
        _stream_add_(z, self.transition_z(z), sd)
        return z


class PairSingleBlock(nn.Module):
    """One Pairformer block with a single track, as the benchmark configs define it.

    Pair track = ``PairformerBlock`` (modules/apo_module.py:145-172); single track =
    the part of ``ConfidencePairSingleBlock.forward`` after its pair block
    (modules/confidence_head.py:161-175): ``bias = linear_pair_bias(LN(z))`` moved to
    [B, H, L, L], ``s += SelfAttentionPairBias(s, None, bias, mask)``,
    ``s += Transition_4(s)``.
    """

    def __init__(self, channel_s: int = 384, channel_z: int = 128, num_heads: int = 16,
                 num_tri_heads: int = 4, row_chunk: int | None = None,
                 stream_dtype: torch.dtype | None = None):
        super().__init__()
        self.stream_dtype = stream_dtype
        self.pair_block = PairformerBlock(channel_z, num_tri_heads, row_chunk=row_chunk,
                                          stream_dtype=stream_dtype)
        self.layernorm_z = LayerNorm(channel_z)
        self.linear_pair_bias = LinearNoBias(channel_z, num_heads)
        self.attention = SelfAttentionPairBias(channel_s, num_heads, None, call_site="confidence")
        self.transition = Transition(channel_s, expansion_factor=4)

    def forward(self, z, s, pair_mask, mask):
        z = self.pair_block(z, pair_mask)
        pair_bias = self.linear_pair_bias(self.layernorm_z(z)).movedim(-1, -3)
        _stream_add_(s, self.attention(s, None, pair_bias, mask), self.stream_dtype)
        _stream_add_(s, self.transition(s), self.stream_dtype)
        return z, s


class PairformerTrunk(nn.Module):
    """A stack of ``PairSingleBlock`` (plain loop at inference, utils/checkpointing.py:85-86)."""

    def __init__(self, num_blocks: int, channel_s: int = 384, channel_z: int = 128,
                 num_heads: int = 16, num_tri_heads: int = 4, row_chunk: int | None = None,
                 stream_dtype: torch.dtype | None = None):
        super().__init__()
        self.blocks = nn.ModuleList(
            PairSingleBlock(channel_s, channel_z, num_heads, num_tri_heads, row_chunk, stream_dtype)
            for _ in range(num_blocks))

    def forward(self, z, s, pair_mask, mask):
        for blk in self.blocks:
            z, s = blk(z, s, pair_mask, mask)
        return z, s


# ---------------------------------------------------------------------------
# Parcae recurrence of the trunk
# ---------------------------------------------------------------------------
class ParcaeStep(nn.Module):
    """model/model.py:201-217 (parameters), :272-277 (discretised dynamics), :523-529 (the step
    ``z = a * z + F.linear(layernorm_z(u), b)``).  fp32 throughout (the reference casts ``a`` and
    ``b`` to its autocast dtype, :505)."""

    def __init__(self, channel_z: int = 256, decay_init: float = 0.9):
        super().__init__()
        self.layernorm_z = LayerNorm(channel_z)
        self.parcae_log_a = nn.Parameter(torch.zeros(channel_z))
        delta_init = -math.log(decay_init)
        self.parcae_log_delta = nn.Parameter(torch.full((channel_z,), math.log(math.expm1(delta_init))))
        self.parcae_b_cont = nn.Parameter(torch.eye(channel_z))

    def dynamics(self):
        delta = F.softplus(self.parcae_log_delta)                    # :274
        a = torch.exp(-delta * torch.exp(self.parcae_log_a))         # :275
        b = delta[:, None] * self.parcae_b_cont                      # :276
        return a, b

    def forward(self, z: torch.Tensor, u: torch.Tensor) -> torch.Tensor:
        a, b = self.dynamics()
        return a * z + F.linear(self.layernorm_z(u), b)              # :528


class TrianglularStack(nn.Module):
    """model/modules/tri_stack.py:31-93 (plain loop at inference)."""

    def __init__(self, channel_z: int = 256, num_blocks: int = 48):
        super().__init__()
        self.blocks = nn.ModuleList(TriangularBlock(channel_z) for _ in range(num_blocks))

    def forward(self, z, pair_mask):
        for blk in self.blocks:
            z = blk(z, pair_mask)
        return z


class ParcaeTrunk(ParcaeStep):
    """The recurrence of ``KFold.run_trunk`` (model/model.py:522-529) with the dropout on ``z_lm``
    (:525) left to the caller."""

    def __init__(self, channel_z: int = 256, lm_blocks: int = 4, main_blocks: int = 48,
                 decay_init: float = 0.4472135954999579):
        super().__init__(channel_z, decay_init)
        self.lm_stack = TrianglularStack(channel_z, lm_blocks)
        self.main_stack = TrianglularStack(channel_z, main_blocks)

    def forward(self, z, z_inputs, z_lm, pair_mask, num_recycles: int = 0):
        a, b = self.dynamics()
        for _ in range(num_recycles + 1):
            u_t = z_inputs + self.lm_stack(z_lm.clone(), pair_mask)              # :526
            z = a * z + F.linear(self.layernorm_z(u_t), b)                        # :528
            z = self.main_stack(z, pair_mask)                                     # :529
        return z
