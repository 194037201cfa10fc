"""Pairformer block / trunk composition on the hip backend.

``PairformerBlock`` mirrors the reference's pair track
(src/kfold/model/modules/apo_module.py:107-172); ``PairSingleBlock`` adds the single track
of ``ConfidencePairSingleBlock.forward`` (model/modules/confidence_head.py:161-175) on top,
which is the block the benchmark configs are quoted on; ``TriangularBlock`` mirrors the
shipping trunk block (model/modules/tri_stack.py:96-151, no triangle attention).

Residual adds are fused into the producing kernels (``z += update`` happens in the output
phase of each op, in place on the caller's tensor like the reference's eval-mode
``z.add_``), and the block's final ``z * pair_mask`` is fused into the transition kernel.
"""

from __future__ import annotations

import torch
from torch import nn

from . import ops
from .layers.attention_pair_bias import SelfAttentionPairBias, _cond_channels, _parameters, norm_eps
from .layers.transition import Transition, hip_transition
from .primitives._common import cache_key, cached_blob, check_inf, check_inference
from .primitives.layers import LayerNorm, LinearNoBias
from .primitives.triangle_attention import (
    TriangleAttentionEndingNode,
    TriangleAttentionStartingNode,
)
from .primitives.triangle_attention import _parameters as _ta_parameters
from .primitives.triangle_multiplication import (
    TriangleMultiplicationIncoming,
    TriangleMultiplicationOutgoing,
)
from .primitives.triangle_multiplication import _parameters as _tm_parameters


def _contiguous_io(t: torch.Tensor, name: str) -> None:
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous for the in-place hip block")
    if t.dtype not in (torch.bfloat16, torch.float32):
        raise TypeError(f"{name}: the hip block runs on bfloat16 or float32 tensors, got {t.dtype}")


def _trimul_inplace(mod: nn.Module, z: torch.Tensor, mask: torch.Tensor, before_write=None,
                    row_chunks: int = 1, side=None) -> None:
    params = _tm_parameters(mod)
    blob = cached_blob(mod, "_hip_multiplication_cache", cache_key(params, z, torch.bfloat16),
                       lambda: ops.trimul_pack(*params, device=z.device))
    ops.trimul_forward(z, mask, blob, mod.direction, eps=mod.layernorm_in.eps, residual=z, out=z,
                       before_write=before_write, row_chunks=row_chunks, side=side)


def _triattn_inplace(mod: nn.Module, z: torch.Tensor, mask: torch.Tensor, row_chunks: int = 1, side=None) -> None:
    check_inf(mod)
    params = _ta_parameters(mod)
    blob = cached_blob(mod, "_hip_attention_cache", cache_key(params, z, torch.bfloat16),
                       lambda: ops.triattn_pack(*params, device=z.device))
    ops.triattn_forward(z, mask, blob, mod.no_heads, mod.starting, eps=mod.layer_norm.eps,
                        residual=z, out=z, row_chunks=row_chunks, side=side)


def _phase_stream(holder: nn.Module, z: torch.Tensor):
    """The second stream of a block that overlaps the phases of its ops (one per block and device)."""
    if z.device.type != "cuda":
        return None
    cached = getattr(holder, "_hip_phase_stream", None)
    if cached is None or cached[0] != z.device:
        cached = (z.device, torch.cuda.Stream(z.device))
        holder._hip_phase_stream = cached
    return cached[1]


class PairformerBlock(nn.Module):
    """tri-mul out, tri-mul in, tri-attn start, tri-attn end, transition(x2), final mask."""

    def __init__(self, channel_z: int = 128, num_tri_heads: int = 4, dropout: float = 0.1,
                 kernel_backend: str = "hip", phase_row_chunks: int = 1):
        super().__init__()
        self.kernel_backend = kernel_backend
        self.channel_z = channel_z
        # > 1: every triangle op runs its contraction / attention and its output phase over that many
        # ranges of rows, the (memory-bound) output phase of a range on a second stream beside the
        # (compute-bound) core phase of the next; results are the same bits (batch 1, c_z = 128)
        self.phase_row_chunks = phase_row_chunks
        self.tri_mul_out = TriangleMultiplicationOutgoing(channel_z, kernel_backend=kernel_backend)
        self.tri_mul_in = TriangleMultiplicationIncoming(channel_z, kernel_backend=kernel_backend)
        self.tri_att_start = TriangleAttentionStartingNode(channel_z, num_tri_heads,
                                                           kernel_backend=kernel_backend)
        self.tri_att_end = TriangleAttentionEndingNode(channel_z, num_tri_heads,
                                                       kernel_backend=kernel_backend)
        self.transition_z = Transition(channel_z, expansion_factor=2)

    def forward(self, z: torch.Tensor, pair_mask: torch.Tensor, inplace_output: bool = False,
                before_first_write=None) -> torch.Tensor:
        """z [B, N, N, C] is updated in place by the four triangle ops (as the reference does in
        eval mode); returns ``(z + transition(z)) * pair_mask`` as a new tensor, or written over
        ``z`` when ``inplace_output`` is set.  ``before_first_write`` is called once, right before
        the first kernel that writes ``z`` is enqueued (see ``PairformerTrunk``)."""
        check_inference(z, "Pairformer block")
        if self.training:
            raise RuntimeError("The hip Pairformer block is inference-only (call .eval()).")
        _contiguous_io(z, "z")
        k = self.phase_row_chunks
        side = _phase_stream(self, z) if k > 1 else None
        _trimul_inplace(self.tri_mul_out, z, pair_mask, before_write=before_first_write, row_chunks=k, side=side)
        _trimul_inplace(self.tri_mul_in, z, pair_mask, row_chunks=k, side=side)
        _triattn_inplace(self.tri_att_start, z, pair_mask, row_chunks=k, side=side)
        _triattn_inplace(self.tri_att_end, z, pair_mask, row_chunks=k, side=side)
        return hip_transition(self.transition_z, z, residual=z, mask=pair_mask,
                              out=z if inplace_output else None)


class TriangularBlock(nn.Module):
    """tri-mul out, tri-mul in, transition(x4); no triangle attention, no final mask."""

    def __init__(self, channel_z: int = 128, dropout: float = 0.25, kernel_backend: str = "hip"):
        super().__init__()
        self.kernel_backend = kernel_backend
        self.channel_z = channel_z
        self.tri_mul_out = TriangleMultiplicationOutgoing(channel_z, kernel_backend=kernel_backend)
        self.tri_mul_in = TriangleMultiplicationIncoming(channel_z, kernel_backend=kernel_backend)
        self.transition_z = Transition(channel_z, expansion_factor=4)

    def forward(self, z: torch.Tensor, pair_mask: torch.Tensor) -> torch.Tensor:
        check_inference(z, "triangular block")
        if self.training:
            raise RuntimeError("The hip triangular block is inference-only (call .eval()).")
        _contiguous_io(z, "z")
        _trimul_inplace(self.tri_mul_out, z, pair_mask)
        _trimul_inplace(self.tri_mul_in, z, pair_mask)
        return hip_transition(self.transition_z, z, residual=z, out=z)


class PairSingleBlock(nn.Module):
    """Pair track (``PairformerBlock``) followed by the single track: pair bias from z,
    ``s += SelfAttentionPairBias(s)``, ``s += Transition_4(s)``."""

    def __init__(self, channel_s: int = 384, channel_z: int = 128, num_heads: int = 16,
                 num_tri_heads: int = 4, kernel_backend: str = "hip"):
        super().__init__()
        self.kernel_backend = kernel_backend
        self.num_heads = num_heads
        self.pair_block = PairformerBlock(channel_z, num_tri_heads, kernel_backend=kernel_backend)
        self.layernorm_z = LayerNorm(channel_z)
        self.linear_pair_bias = LinearNoBias(channel_z, num_heads)
        self.attention = SelfAttentionPairBias(channel_s, num_heads, None, call_site="confidence",
                                               kernel_backend=kernel_backend)
        self.transition = Transition(channel_s, expansion_factor=4)

    def forward(self, z: torch.Tensor, s: torch.Tensor, pair_mask: torch.Tensor, mask: torch.Tensor,
                inplace_output: bool = False):
        """z [B, N, N, Cz], s [B, N, Cs], pair_mask [B, N, N], mask [B, N]; s is updated in place."""
        _contiguous_io(s, "s")
        z = self.pair_block(z, pair_mask, inplace_output=inplace_output)
        self.single_track(z, s, mask)
        return z, s

    def single_track(self, z: torch.Tensor, s: torch.Tensor, mask: torch.Tensor, after_bias=None) -> None:
        """``s += SelfAttentionPairBias(s; bias(z))``, ``s += Transition_4(s)`` on the current stream.
        ``after_bias`` is called once the last kernel that reads ``z`` has been enqueued."""
        B = z.shape[0]
        if s.numel() == 0:                  # no tokens: nothing to update
            if after_bias is not None:
                after_bias()
            return
        pb_params = (self.layernorm_z.weight, self.layernorm_z.bias, self.linear_pair_bias.weight)
        pb_blob = cached_blob(self, "_hip_pair_bias_cache", cache_key(pb_params, z, torch.bfloat16),
                              lambda: ops.pair_bias_pack(*pb_params, device=z.device))
        tiles = ops.pair_bias_project(z, pb_blob, self.num_heads, eps=self.layernorm_z.eps)
        if after_bias is not None:
            after_bias()
        att = self.attention
        check_inf(att)
        params = _parameters(att)
        blob = cached_blob(att, "_hip_apb_cache", cache_key(tuple(params.values()), s, torch.bfloat16),
                           lambda: ops.apb_pack(att.channel_a, att.num_heads, _cond_channels(att),
                                                device=s.device, **params))
        ops.apb_forward(s, None, tiles, mask.reshape(B, -1), blob, att.num_heads, 0, True, B > 1,
                        eps=norm_eps(att), residual=s, out=s)
        hip_transition(self.transition, s, residual=s, out=s)


class PairformerTrunk(nn.Module):
    """A stack of ``PairSingleBlock``; z and s are updated in place block after block.

    With ``overlap_tracks`` (default) the single track of block b runs on a second HIP stream
    while the pair track of block b+1 runs on the caller's stream: the single track only reads
    the final ``z`` of its block (for the pair bias), and the next pair track never touches ``s``.
    Events keep the reference's order of effects: the single track starts after its block's last
    write of ``z``, and the next block's first write of ``z`` waits until the pair-bias kernel has
    read it.  Both streams have the default priority.  The result is bit-identical to the serial
    schedule."""

    def __init__(self, num_blocks: int, channel_s: int = 384, channel_z: int = 128,
                 num_heads: int = 16, num_tri_heads: int = 4, kernel_backend: str = "hip",
                 overlap_tracks: bool = True):
        super().__init__()
        self.overlap_tracks = overlap_tracks
        self.blocks = nn.ModuleList(
            PairSingleBlock(channel_s, channel_z, num_heads, num_tri_heads, kernel_backend)
            for _ in range(num_blocks))
        self._side = {}

    def _side_stream(self, device: torch.device) -> torch.cuda.Stream:
        key = (device.type, device.index)
        if key not in self._side:
            self._side[key] = torch.cuda.Stream(device=device)
        return self._side[key]

    def forward(self, z, s, pair_mask, mask):
        return run_blocks(list(self.blocks), z, s, pair_mask, mask,
                          self._side_stream(z.device) if self.overlap_tracks and z.is_cuda else None)


def run_blocks(blocks, z, s, pair_mask, mask, side: "torch.cuda.Stream | None" = None):
    """Apply ``PairSingleBlock``s in turn to (z, s), in place.  With a ``side`` stream the single
    tracks run there, overlapped with the following block's pair track (see ``PairformerTrunk``)."""
    if side is None or len(blocks) == 0:
        for blk in blocks:
            z, s = blk(z, s, pair_mask, mask, inplace_output=True)
        return z, s
    _contiguous_io(s, "s")
    main = torch.cuda.current_stream(z.device)
    side.wait_stream(main)                     # s (and the weights) may have been produced on main
    z_read = None                              # event: the previous block's pair-bias kernel has read z
    for blk in blocks:
        wait = None
        if z_read is not None:
            ev = z_read
            wait = lambda ev=ev: main.wait_event(ev)
        z = blk.pair_block(z, pair_mask, inplace_output=True, before_first_write=wait)
        z_done = torch.cuda.Event()
        z_done.record(main)
        z_read = torch.cuda.Event()
        with torch.cuda.stream(side):
            side.wait_event(z_done)
            blk.single_track(z, s, mask, after_bias=lambda ev=z_read: ev.record(side))
    main.wait_stream(side)
    return z, s


class ParcaeStep(nn.Module):
    """The trunk's Parcae recurrence ``z <- a * z + B LN(u)`` (reference:
    src/kfold/model/model.py:523-529; parameters named as on ``KFold``, :201-217:
    ``layernorm_z``, ``parcae_log_a``, ``parcae_log_delta``, ``parcae_b_cont``).  One fused kernel;
    ``z`` is updated in place unless ``inplace=False``."""

    def __init__(self, channel_z: int = 256, decay_init: float = 0.9, kernel_backend: str = "hip"):
        super().__init__()
        import math

        self.kernel_backend = kernel_backend
        self.channel_z = channel_z
        self.layernorm_z = LayerNorm(channel_z)
        self.parcae_log_a = nn.Parameter(torch.zeros(channel_z))
        delta_init = -math.log(decay_init)
        self.parcae_log_delta = nn.Parameter(torch.full((channel_z,), math.log(math.expm1(delta_init))))
        self.parcae_b_cont = nn.Parameter(torch.eye(channel_z))

    def forward(self, z: torch.Tensor, u: torch.Tensor, inplace: bool = True,
                u_add: torch.Tensor | None = None) -> torch.Tensor:
        """``a * z + B LN(u [+ u_add])``."""
        check_inference(z, "Parcae step")
        _contiguous_io(z, "z")
        params = (self.layernorm_z.weight, self.layernorm_z.bias, self.parcae_log_a, self.parcae_log_delta,
                  self.parcae_b_cont)
        blob = cached_blob(self, "_hip_parcae_cache", cache_key(params, z, torch.bfloat16),
                           lambda: ops.parcae_pack(*params, device=z.device))
        return ops.parcae_step(z, u.contiguous(), blob, eps=self.layernorm_z.eps, out=z if inplace else None,
                               u_add=u_add)


class TrianglularStack(nn.Module):
    """A stack of ``TriangularBlock`` (reference: model/modules/tri_stack.py:31-93, same spelling
    and the same ``blocks`` list, so its state-dict keys are the reference's)."""

    def __init__(self, channel_z: int = 256, num_blocks: int = 48, dropout: float = 0.25,
                 blocks_per_ckpt: int | None = None, kernel_backend: str = "hip"):
        super().__init__()
        self.kernel_backend = kernel_backend
        self.channel_z = channel_z
        self.num_blocks = num_blocks
        self.blocks = nn.ModuleList(TriangularBlock(channel_z, dropout, kernel_backend=kernel_backend)
                                    for _ in range(num_blocks))

    def forward(self, z: torch.Tensor, pair_mask: torch.Tensor) -> torch.Tensor:
        """z is updated in place block after block (the reference's eval-mode adds)."""
        for blk in self.blocks:
            z = blk(z, pair_mask)
        return z


class ParcaeTrunk(ParcaeStep):
    """The pair-state recurrence of ``KFold.run_trunk`` (model/model.py:522-529) on the hip backend:

        for each recycle:  u = z_inputs + lm_stack(z_lm);  z = a * z + B LN(u);  z = main_stack(z)

    Sub-modules and parameters carry the names they have on the reference's ``KFold`` (``lm_stack``,
    ``main_stack``, ``layernorm_z``, ``parcae_log_a``, ``parcae_log_delta``, ``parcae_b_cont``), so
    ``load_reference_weights`` fills them from a KFold state dict.  The reference draws a fresh
    dropout mask on ``z_lm`` every recycle (:525); pass the already dropped-out tensor (or a
    callable returning it) as ``z_lm``."""

    def __init__(self, channel_z: int = 256, lm_blocks: int = 4, main_blocks: int = 48,
                 decay_init: float = 0.4472135954999579, kernel_backend: str = "hip"):
        super().__init__(channel_z, decay_init, kernel_backend)
        self.lm_stack = TrianglularStack(channel_z, lm_blocks, kernel_backend=kernel_backend)
        self.main_stack = TrianglularStack(channel_z, main_blocks, kernel_backend=kernel_backend)

    def forward(self, z: torch.Tensor, z_inputs: torch.Tensor, z_lm, pair_mask: torch.Tensor,
                num_recycles: int = 0) -> torch.Tensor:
        """z [B, N, N, C] (the pair state, updated in place), z_inputs [B, N, N, C], z_lm a tensor
        or a callable giving this recycle's (dropped-out) LM pair embedding."""
        for _ in range(num_recycles + 1):
            lm_in = z_lm() if callable(z_lm) else z_lm
            lm = self.lm_stack(lm_in.clone(), pair_mask)          # the stack works in place
            ParcaeStep.forward(self, z, lm, inplace=True, u_add=z_inputs.contiguous())
            z = self.main_stack(z, pair_mask)
        return z
