"""Self attention with pair bias, ``hip`` backend.

``SelfAttentionPairBias`` mirrors the reference module
(src/kfold/model/layers/folding/attention_pair_bias.py:70-158; parameters of
``AttentionPairBias`` :30-67 and ``AdaLN`` model/primitives/normalization.py:94-115).
``hip_attention_pair_bias`` is what a ``kernel_backend == "hip"`` branch of
``attention_pair_bias`` (model/primitives/attention.py:62-66) would call, next to
``triton_attention_pair_bias``: it receives already normalised ``x_q``/``x_k``.

``CrossAttentionPairBias`` mirrors the local-window attention of the atom transformer
(:161-260): Lq queries against Lk keys per window, one bias and key mask per window.

Arithmetic.  The reference runs its trunk and confidence head under bf16 autocast
(inference/runner.py:565-571) and its diffusion stack outside it, on fp32 tensors with full
fp32 dot products (model/model.py:419, kernels/triton/attention_pair_bias/dispatch.py:439,453).
The modules here follow that: ``arith = "auto"`` (the default) selects the library's fp32
arithmetic (``KFH_ARITH_F32``) for a diffusion call site when the activations are fp32 and
autocast is off, and bf16 arithmetic everywhere else; ``"bf16"`` / ``"f32"`` force one.
"""

from __future__ import annotations

import torch
from torch import nn

from .. import ops
from ..primitives._common import cache_key, cached_blob, check_inf, check_inference
from ..primitives.layers import LayerNorm, Linear, LinearNoBias


def _parameters(module: nn.Module):
    cond = getattr(module, "use_single_conditioning", False)
    p = dict(q_w=module.linear_q.weight, q_b=module.linear_q.bias, k_w=module.linear_k.weight,
             v_w=module.linear_v.weight, g_w=module.linear_g.weight, o_w=module.linear_out.weight)
    if cond:
        ada = module.adaln_a
        p.update(adaln_s_w=ada.layernorm_s.weight, adaln_g_w=ada.linear_g.weight,
                 adaln_g_b=ada.linear_g.bias, adaln_bias_w=ada.linear_bias.weight,
                 ada_out_w=module.linear_ada_out.weight, ada_out_b=module.linear_ada_out.bias)
    elif hasattr(module, "layernorm_a"):
        p.update(ln_w=module.layernorm_a.weight, ln_b=module.layernorm_a.bias)
    return p


def _cond_channels(module: nn.Module) -> int:
    if getattr(module, "use_single_conditioning", False):
        return module.linear_ada_out.weight.shape[1]
    return 0


def norm_eps(module: nn.Module) -> float:
    """The one LayerNorm epsilon the fused entry point takes: ``layernorm_a.eps``, or for the
    conditioned module the common value of AdaLN's two LayerNorms."""
    if getattr(module, "use_single_conditioning", False):
        ea, es = module.adaln_a.layernorm_a.eps, module.adaln_a.layernorm_s.eps
        if ea != es:
            raise NotImplementedError(f"hip AdaLN: layernorm_a.eps ({ea}) != layernorm_s.eps ({es})")
        return ea
    return module.layernorm_a.eps if hasattr(module, "layernorm_a") else 1e-5


def select_arith(module: nn.Module, x: torch.Tensor, call_site: str | None = None) -> int:
    """``call_site``: the one the caller names (the functional entry), else the module's own."""
    mode = getattr(module, "arith", "auto")
    if mode == "f32":
        return ops.KFH_ARITH_F32
    if mode == "bf16":
        return ops.KFH_ARITH_BF16
    if mode != "auto":
        raise ValueError(f"arith must be 'auto', 'bf16' or 'f32', got {mode!r}")
    site = call_site if call_site is not None else getattr(module, "call_site", "diffusion_local")
    diffusion = str(site).startswith("diffusion")
    if diffusion and x.dtype == torch.float32 and not torch.is_autocast_enabled():
        return ops.KFH_ARITH_F32
    return ops.KFH_ARITH_BF16


class PairBiasTiles:
    """A pair bias already in the attention kernel's tile order.

    The diffusion sampler computes the pair bias of every transformer block once and uses it at
    every step (model/modules/ecsi.py:506-512); converting the dense ``[*, H, L, L]`` tensor to tiles
    on each call re-reads and re-writes it every time.  ``prepare_pair_bias`` does the conversion once;
    the result is accepted wherever the self-attention entries take ``pair_bias``."""

    def __init__(self, tiles: torch.Tensor, lead: tuple, heads: int, length: int, arith: int):
        self.tiles, self.lead, self.heads, self.length, self.arith = tiles, tuple(lead), heads, length, arith

    @property
    def shape(self):
        return self.lead + (self.heads, self.length, self.length)


def prepare_pair_bias(pair_bias: torch.Tensor, arith: str | int = "bf16") -> PairBiasTiles:
    """Dense pair bias ``[*, H, L, L]`` -> tiles for the arithmetic the attention will run in
    ("bf16" or "f32": what ``select_arith`` gives for the call; a mismatch raises at the call)."""
    if isinstance(arith, str):
        if arith not in ("bf16", "f32"):
            raise ValueError(f"arith must be 'bf16' or 'f32', got {arith!r}")
        arith = ops.KFH_ARITH_F32 if arith == "f32" else ops.KFH_ARITH_BF16
    if pair_bias.dim() < 3 or pair_bias.shape[-1] != pair_bias.shape[-2]:
        raise ValueError(f"expected pair_bias [*, H, L, L], got {tuple(pair_bias.shape)}")
    lead = tuple(pair_bias.shape[:-3])
    flat = pair_bias.reshape((-1,) + pair_bias.shape[-3:])
    return PairBiasTiles(ops.bias_tiles_from_dense(flat, arith), lead, pair_bias.shape[-3], pair_bias.shape[-1], arith)


def _bias_tiles(pair_bias, lead: torch.Size, arith: int, heads: int, length: int):
    """(tiles, one bias per flattened sample?) for a dense or a prepared pair bias."""
    if isinstance(pair_bias, PairBiasTiles):
        if pair_bias.arith != arith:
            raise ValueError("the pair bias was prepared for the other arithmetic "
                             f"({'f32' if pair_bias.arith == ops.KFH_ARITH_F32 else 'bf16'})")
        if pair_bias.heads != heads or pair_bias.length != length:
            raise ValueError(f"prepared pair bias {pair_bias.shape} does not match {heads} heads x {length} tokens")
        n = 1
        for d in pair_bias.lead:
            n *= d
        full = 1
        for d in lead:
            full *= d
        if n == 1:
            return pair_bias.tiles, False
        if tuple(pair_bias.lead) != tuple(lead)[-len(pair_bias.lead):] or n != full:
            raise ValueError(f"prepared pair bias {pair_bias.shape} must have one bias in all or the "
                             f"leading dims {tuple(lead)} of the activations")
        return pair_bias.tiles, True
    pb, per_sample = _flatten(pair_bias, 3, lead)
    return ops.bias_tiles_from_dense(pb, arith), per_sample


def _flatten(t: torch.Tensor, keep: int, lead: torch.Size):
    """Flatten the leading dims of ``t`` (which broadcast against ``lead``) to 1 or prod(lead)."""
    tl = t.shape[:t.dim() - keep]
    if all(d == 1 for d in tl):
        return t.reshape((1,) + t.shape[t.dim() - keep:]), False
    full = torch.broadcast_to(t, tuple(lead) + t.shape[t.dim() - keep:])
    return full.reshape((-1,) + t.shape[t.dim() - keep:]), True


def _run(module, a, s, pair_bias, mask, apply_norm: bool, call_site: str | None = None) -> torch.Tensor:
    check_inference(a, "pair-bias attention")
    check_inf(module)
    if module.linear_g.bias is not None or module.linear_out.bias is not None:
        raise NotImplementedError("hip pair-bias attention: gate / output projection biases")
    if a.numel() == 0:                      # no samples or no tokens: nothing to attend to
        return torch.empty_like(a)
    params = _parameters(module)
    C, H, Cs = module.channel_a, module.num_heads, _cond_channels(module)
    arith = select_arith(module, a, call_site)
    key = cache_key(tuple(params.values()), a,
                    torch.float32 if arith == ops.KFH_ARITH_F32 else torch.bfloat16)
    blob = cached_blob(module, "_hip_apb_cache", key,
                       lambda: ops.apb_pack(C, H, Cs, device=a.device, arith=arith, **params))
    lead = a.shape[:-2]
    io = a if a.dtype in (torch.bfloat16, torch.float32) else a.float()
    af = io.reshape((-1,) + a.shape[-2:])
    tiles, per_sample = _bias_tiles(pair_bias, lead, arith, H, a.shape[-2])
    mk, _ = _flatten(mask, 1, lead)
    sf = None
    if s is not None and apply_norm and Cs:
        sf, _ = _flatten(s, 2, lead)
    out = ops.apb_forward(af, sf, tiles, mk, blob, H, Cs, apply_norm, per_sample and af.shape[0] > 1,
                          eps=norm_eps(module), arith=arith)
    return out.reshape(a.shape).to(a.dtype)


def _run_cross(module, x_q, x_k, pair_bias, mask, call_site: str | None = None) -> torch.Tensor:
    """Already normalised queries x_q [*, Lq, C] against keys x_k [*, Lk, C]: q/k/v/gate/output
    projections and the attention only (the caller has normalised and applies its own
    conditioning gate afterwards, attention_pair_bias.py:241-262 of the reference)."""
    check_inference(x_q, "cross attention with pair bias")
    check_inf(module)
    if module.linear_g.bias is not None or module.linear_out.bias is not None:
        raise NotImplementedError("hip cross attention: gate / output projection biases")
    if x_q.numel() == 0:                    # no windows or no queries
        return torch.empty_like(x_q)
    w = dict(q_w=module.linear_q.weight, q_b=module.linear_q.bias, k_w=module.linear_k.weight,
             v_w=module.linear_v.weight, g_w=module.linear_g.weight, o_w=module.linear_out.weight)
    arith = select_arith(module, x_q, call_site)
    C, H = module.channel_a, module.num_heads
    key = cache_key(tuple(w.values()), x_q, torch.float32 if arith == ops.KFH_ARITH_F32 else torch.bfloat16)
    blob = cached_blob(module, "_hip_cross_functional_cache", key,
                       lambda: ops.cross_apb_pack(C, H, 0, x_q.device, arith=arith, **w))
    lead = x_q.shape[:-2]
    Lq = x_q.shape[-2]
    io = x_q if x_q.dtype in (torch.bfloat16, torch.float32) else x_q.float()

    def flat(t, keep):
        full = torch.broadcast_to(t, tuple(lead) + t.shape[t.dim() - keep:])
        return full.reshape((-1,) + t.shape[t.dim() - keep:])

    out = ops.cross_apb_forward(io.reshape(-1, Lq, C), flat(x_k, 2), None, None, flat(pair_bias, 3),
                                flat(mask, 1), blob, H, 0, apply_norm=False, arith=arith)
    return out.reshape(x_q.shape).to(x_q.dtype)


@torch.compiler.disable
def hip_attention_pair_bias(module: nn.Module, x_q: torch.Tensor, x_k: torch.Tensor,
                            pair_bias: torch.Tensor, mask: torch.Tensor, *,
                            call_site: str = "confidence") -> torch.Tensor:
    """x_q [*, Lq, C], x_k [*, Lk, C] normalised, pair_bias broadcastable to [*, H, Lq, Lk], mask
    broadcastable to [*, Lk] (the signature of model/primitives/attention.py:28-37).  The same
    tensor on both sides is self attention; different tensors are the local windows of
    ``CrossAttentionPairBias`` (call site "diffusion_local")."""
    if x_q is not x_k and (x_q.shape != x_k.shape or x_q.data_ptr() != x_k.data_ptr()
                           or x_q.stride() != x_k.stride()):
        return _run_cross(module, x_q, x_k, pair_bias, mask, call_site)
    return _run(module, x_q, None, pair_bias, mask, apply_norm=False, call_site=call_site)


class AdaLN(nn.Module):
    """Parameter holder, names of model/primitives/normalization.py:94-115."""

    def __init__(self, channel_a: int, channel_s: int):
        super().__init__()
        self.layernorm_a = LayerNorm(channel_a, create_scale=False, create_offset=False)
        self.layernorm_s = LayerNorm(channel_s, create_scale=True, create_offset=False)
        self.linear_g = Linear(channel_s, channel_a, init="gating")
        self.linear_bias = LinearNoBias(channel_s, channel_a, init="final")


class SelfAttentionPairBias(nn.Module):
    def __init__(self, channel_a: int, num_heads: int, channel_s: int | None, call_site: str,
                 inf: float = 1e9, kernel_backend: str = "hip", arith: str = "auto") -> None:
        super().__init__()
        if kernel_backend != "hip":
            raise ValueError(
                f"kfold_amd implements kernel_backend='hip' only, got {kernel_backend!r}")
        if call_site not in {"diffusion_global", "confidence"}:
            raise ValueError(f"Unsupported self APB call site: {call_site!r}")
        self.arith = arith
        assert channel_a % num_heads == 0
        self.use_single_conditioning = channel_s is not None
        self.call_site = call_site
        self.channel_a = channel_a
        self.num_heads = num_heads
        self.head_dim = channel_a // num_heads
        self.inf = inf
        self.kernel_backend = kernel_backend
        self.linear_q = Linear(channel_a, channel_a, init="default")
        self.linear_k = LinearNoBias(channel_a, channel_a, init="default")
        self.linear_v = LinearNoBias(channel_a, channel_a, init="default")
        self.linear_g = LinearNoBias(channel_a, channel_a, init="gating")
        self.linear_out = LinearNoBias(channel_a, channel_a,
                                       init="default" if self.use_single_conditioning else "final")
        if self.use_single_conditioning:
            self.adaln_a = AdaLN(channel_a, channel_s)
            self.linear_ada_out = Linear(channel_s, channel_a, init="gating")
            with torch.no_grad():
                self.linear_ada_out.bias.fill_(-2.0)      # the reference's "gating_closed"
        else:
            self.layernorm_a = LayerNorm(channel_a, create_offset=True)

    def forward(self, a: torch.Tensor, s: torch.Tensor | None, pair_bias: torch.Tensor,
                mask: torch.Tensor) -> torch.Tensor:
        """a [..., L, c_a], s [..., L, c_s] or None, pair_bias [..., H, L, L], mask [..., L]."""
        if self.use_single_conditioning:
            assert s is not None
        else:
            assert s is None
        return _run(self, a, s, pair_bias, mask, apply_norm=True)


class CrossAttentionPairBias(nn.Module):
    """Mirror of the reference's ``CrossAttentionPairBias`` (attention_pair_bias.py:161-260): same
    constructor, parameter names (``layernorm_a_q`` / ``layernorm_a_k`` or ``adaln_a_q`` /
    ``adaln_a_k`` + ``linear_ada_out``) and ``forward(a_q, a_k, s_q, s_k, pair_bias, mask)``."""

    def __init__(self, channel_a: int, num_heads: int, channel_s: int | None, inf: float = 1e9,
                 kernel_backend: str = "hip", arith: str = "auto") -> None:
        super().__init__()
        if kernel_backend != "hip":
            raise ValueError(f"kfold_amd implements kernel_backend='hip' only, got {kernel_backend!r}")
        assert channel_a % num_heads == 0
        self.arith = arith
        self.call_site = "diffusion_local"
        self.use_single_conditioning = channel_s is not None
        self.channel_a = channel_a
        self.channel_s = channel_s
        self.num_heads = num_heads
        self.head_dim = channel_a // num_heads
        self.inf = inf
        self.kernel_backend = kernel_backend
        self.linear_q = Linear(channel_a, channel_a, init="default")
        self.linear_k = LinearNoBias(channel_a, channel_a, init="default")
        self.linear_v = LinearNoBias(channel_a, channel_a, init="default")
        self.linear_g = LinearNoBias(channel_a, channel_a, init="gating")
        self.linear_out = LinearNoBias(channel_a, channel_a,
                                       init="default" if self.use_single_conditioning else "final")
        if self.use_single_conditioning:
            self.adaln_a_q = AdaLN(channel_a, channel_s)
            self.adaln_a_k = AdaLN(channel_a, channel_s)
            self.linear_ada_out = Linear(channel_s, channel_a, init="gating")
            with torch.no_grad():
                self.linear_ada_out.bias.fill_(-2.0)      # the reference's "gating_closed"
        else:
            self.layernorm_a_q = LayerNorm(channel_a, create_offset=True)
            self.layernorm_a_k = LayerNorm(channel_a, create_offset=True)

    def _weights(self) -> dict:
        p = dict(q_w=self.linear_q.weight, q_b=self.linear_q.bias, k_w=self.linear_k.weight,
                 v_w=self.linear_v.weight, g_w=self.linear_g.weight, o_w=self.linear_out.weight)
        if self.use_single_conditioning:
            q, k = self.adaln_a_q, self.adaln_a_k
            p.update(adaq_s_w=q.layernorm_s.weight, adaq_g_w=q.linear_g.weight, adaq_g_b=q.linear_g.bias,
                     adaq_bias_w=q.linear_bias.weight, adak_s_w=k.layernorm_s.weight,
                     adak_g_w=k.linear_g.weight, adak_g_b=k.linear_g.bias, adak_bias_w=k.linear_bias.weight,
                     ada_out_w=self.linear_ada_out.weight, ada_out_b=self.linear_ada_out.bias)
        else:
            p.update(lnq_w=self.layernorm_a_q.weight, lnq_b=self.layernorm_a_q.bias,
                     lnk_w=self.layernorm_a_k.weight, lnk_b=self.layernorm_a_k.bias)
        return p

    @torch.compiler.disable
    def forward(self, a_q: torch.Tensor, a_k: torch.Tensor, s_q: torch.Tensor | None,
                s_k: torch.Tensor | None, pair_bias: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
        """a_q [..., W, Lq, c_a], a_k [..., W, Lk, c_a], s_q / s_k [..., W, L., c_s] or None,
        pair_bias [..., W, H, Lq, Lk], mask [..., W, Lk] -> [..., W, Lq, c_a]."""
        check_inference(a_q, "cross attention with pair bias")
        check_inf(self)
        if self.use_single_conditioning:
            assert s_q is not None and s_k is not None
        else:
            assert s_q is None and s_k is None
        if self.linear_g.bias is not None or self.linear_out.bias is not None:
            raise NotImplementedError("hip cross attention: gate / output projection biases")
        if a_q.numel() == 0:                # no windows or no queries
            return torch.empty_like(a_q)
        w = self._weights()
        cs = self.channel_s or 0
        arith = select_arith(self, a_q)
        key = cache_key(tuple(w.values()), a_q, torch.float32 if arith == ops.KFH_ARITH_F32 else torch.bfloat16)
        blob = cached_blob(self, "_hip_cross_cache", key,
                           lambda: ops.cross_apb_pack(self.channel_a, self.num_heads, cs, a_q.device,
                                                      arith=arith, **w))
        lead = a_q.shape[:-2]
        Lq, Lk = a_q.shape[-2], a_k.shape[-2]
        io = a_q if a_q.dtype in (torch.bfloat16, torch.float32) else a_q.float()

        def flat(t, keep):
            full = torch.broadcast_to(t, tuple(lead) + t.shape[t.dim() - keep:])
            return full.reshape((-1,) + t.shape[t.dim() - keep:])

        eps = (self.adaln_a_q.layernorm_a.eps if self.use_single_conditioning else self.layernorm_a_q.eps)
        out = ops.cross_apb_forward(io.reshape(-1, Lq, self.channel_a), flat(a_k, 2),
                                    None if s_q is None else flat(s_q, 2), None if s_k is None else flat(s_k, 2),
                                    flat(pair_bias, 3), flat(mask, 1), blob, self.num_heads, cs, eps=eps,
                                    arith=arith)
        return out.reshape(a_q.shape).to(a_q.dtype)
