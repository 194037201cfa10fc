"""Host-side plumbing of the hip backend, run without a GPU.

The library handle is replaced by a recorder that checks every call against the ctypes signature
table (argument count and types), answers the size queries with the real library (they need no
GPU) and records the converted arguments instead of launching anything.  What is checked here is
what the Python layer decides: which entry points run in which order, which tensors alias, which
flags, sizes and eps values are passed, when weights are repacked.  Nothing is computed, so these
tests say nothing about numerics; the GPU tests do."""

import contextlib
import sys

import pytest
import torch


class Recorder:
    def __init__(self, real, signatures):
        self.real, self.signatures, self.calls = real, signatures, []

    def __getattr__(self, name):
        res, argtypes = self.signatures[name]              # KeyError: not in the header
        if name.endswith(("_bytes", "_granule")) or name in ("kfh_version", "kfh_last_error"):
            return getattr(self.real, name)

        def call(*args):
            assert len(args) == len(argtypes), f"{name}: {len(args)} arguments, header has {len(argtypes)}"
            conv = tuple(None if a is None else t(a).value for a, t in zip(args, argtypes))
            self.calls.append((name, conv))
            return 0
        return call

    def names(self, suffixes=("_forward", "_forward_stages", "_project", "_step", "_from_dense")):
        return [n for n, _ in self.calls if n.endswith(suffixes)]

    def of(self, name):
        return [a for n, a in self.calls if n == name]


@pytest.fixture
def rec(monkeypatch):
    from kfold_amd import _lib, layers, modules, ops, primitives  # noqa: F401  (patched below)

    r = Recorder(_lib.lib(), _lib.SIGNATURES)
    monkeypatch.setattr(_lib, "lib", lambda: r)

    def any_device(*tensors):
        for t in tensors:
            if t is not None:
                return t.device
    monkeypatch.setattr(ops, "_require_cuda", any_device)
    monkeypatch.setattr(ops, "_stream", lambda dev: 0)
    monkeypatch.setattr(torch.cuda, "device", lambda dev: contextlib.nullcontext())

    def grad_only(x, what):
        if torch.is_grad_enabled():
            raise RuntimeError(f"The hip {what} backend is inference-only.")
    for name, mod in list(sys.modules.items()):
        if name.startswith("kfold_amd") and hasattr(mod, "check_inference"):
            monkeypatch.setattr(mod, "check_inference", grad_only)
    return r


def _inside(ptr, t):
    return t.data_ptr() <= ptr < t.data_ptr() + max(t.numel() * t.element_size(), 1)


def test_pair_single_block_call_sequence_and_aliasing(rec):
    from kfold_amd import modules, ops

    N = 8
    blk = modules.PairSingleBlock().eval()
    blk.pair_block.tri_mul_in.layernorm_in.eps = 3e-5
    blk.pair_block.tri_att_end.layer_norm.eps = 7e-6
    z = torch.zeros(1, N, N, 128, dtype=torch.bfloat16)
    s = torch.zeros(1, N, 384, dtype=torch.bfloat16)
    tok = torch.ones(1, N, dtype=torch.bool)
    tok[:, -2:] = False
    pair = tok[:, :, None] & tok[:, None, :]
    with torch.no_grad():
        z_out, s_out = blk(z, s, pair, tok, inplace_output=True)
    assert z_out.data_ptr() == z.data_ptr() and s_out.data_ptr() == s.data_ptr()
    assert rec.names() == ["kfh_trimul_forward", "kfh_trimul_forward", "kfh_triattn_forward",
                           "kfh_triattn_forward", "kfh_transition_forward", "kfh_pair_bias_project",
                           "kfh_apb_forward", "kfh_transition_forward"]
    out_call, in_call = rec.of("kfh_trimul_forward")
    for c, direction, eps in ((out_call, 0, 1e-5), (in_call, 1, 3e-5)):
        x, mask, blob, resid, out, ws, ws_bytes, B, n, C, d, e, io, stream = c
        assert x == resid == out == z.data_ptr(), "tri-mul runs in place on z with the residual fused"
        assert (B, n, C, d, io) == (1, N, 128, direction, 0)
        assert e == pytest.approx(eps)
        assert ws_bytes == ops.workspace_bytes("trimul", N=N, C=128) and ws
    start, end = rec.of("kfh_triattn_forward")
    assert start[11] == 0 and end[11] == 1, "starting node first, then the ending node"
    assert start[12] == pytest.approx(1e-5) and end[12] == pytest.approx(7e-6)
    assert start[0] == start[3] == start[4] == z.data_ptr()
    pair_tr, single_tr = rec.of("kfh_transition_forward")
    assert pair_tr[0] == pair_tr[2] == pair_tr[4] == z.data_ptr() and pair_tr[3], "final mask fused"
    assert (pair_tr[7], pair_tr[8], pair_tr[9]) == (N * N, 128, 2)
    assert single_tr[0] == single_tr[2] == single_tr[4] == s.data_ptr() and single_tr[3] is None
    assert (single_tr[7], single_tr[8], single_tr[9]) == (N, 384, 4)
    apb = rec.of("kfh_apb_forward")[0]
    assert apb[0] == apb[5] == apb[6] == s.data_ptr() and apb[1] is None
    assert apb[9:14] == (1, N, 384, 16, 0)
    # the mask bytes handed to the kernels hold the pair mask
    packs = [n for n, _ in rec.calls if n.endswith("_pack")]
    assert sorted(packs) == sorted(["kfh_trimul_pack"] * 2 + ["kfh_triattn_pack"] * 2 + ["kfh_transition_pack"] * 2
                                   + ["kfh_pair_bias_pack", "kfh_apb_pack"])


def test_packed_weights_are_cached_until_a_parameter_changes(rec):
    from kfold_amd import primitives

    mod = primitives.TriangleMultiplicationOutgoing(128).eval()
    x = torch.zeros(1, 4, 4, 128, dtype=torch.bfloat16)
    m = torch.ones(1, 4, 4, dtype=torch.bool)
    with torch.no_grad():
        mod(x, m)
        mod(x, m)
        assert len(rec.of("kfh_trimul_pack")) == 1 and len(rec.of("kfh_trimul_forward")) == 2
        mod.linear_p_out.weight.add_(1.0)                      # in-place update bumps the version
        mod(x, m)
        assert len(rec.of("kfh_trimul_pack")) == 2
        mod.load_state_dict({k: v.clone() for k, v in mod.state_dict().items()})
        mod(x, m)
        assert len(rec.of("kfh_trimul_pack")) == 3
    # module-level forward is out of place: z is read, a new tensor is written, no residual
    c = rec.of("kfh_trimul_forward")[-1]
    assert c[0] == x.data_ptr() and c[3] is None and c[4] != x.data_ptr()


def test_caller_workspace_is_used_and_checked(rec):
    from kfold_amd import ops

    N = 8
    z = torch.zeros(1, N, N, 128, dtype=torch.bfloat16)
    m = torch.ones(1, N, N, dtype=torch.bool)
    need_tm = ops.workspace_bytes("trimul", N=N, C=128)
    need_ta = ops.workspace_bytes("triattn", N=N, C=128, heads=4)
    assert need_tm > 0 and need_ta > 0
    assert ops.workspace_bytes("trimul", N=N, C=48) == 0 and ops.workspace_bytes("trimul", N=N, C=64) > 0
    with pytest.raises(ValueError):
        ops.workspace_bytes("softmax", N=N)
    blob = torch.zeros(16, dtype=torch.uint8)
    base = torch.zeros(max(need_tm, need_ta) + 512, dtype=torch.uint8)
    off = (-base.data_ptr()) % 256
    ws = base[off:off + max(need_tm, need_ta)]
    ops.trimul_forward(z, m, blob, "outgoing", workspace=ws)
    ops.triattn_forward(z, m, blob, 4, True, workspace=ws)
    assert rec.of("kfh_trimul_forward")[0][5] == ws.data_ptr()
    assert rec.of("kfh_triattn_forward")[0][5] == ws.data_ptr()
    assert rec.of("kfh_trimul_forward")[0][6] == need_tm and rec.of("kfh_triattn_forward")[0][6] == need_ta
    with pytest.raises(ValueError, match="needs"):
        ops.trimul_forward(z, m, blob, "outgoing", workspace=ws[:need_tm - 256])
    with pytest.raises(ValueError, match="aligned"):
        ops.trimul_forward(z, m, blob, "outgoing", workspace=base[off + 16:off + 16 + need_tm])
    with pytest.raises(ValueError, match="uint8"):
        ops.trimul_forward(z, m, blob, "outgoing", workspace=torch.zeros(need_tm, dtype=torch.int8))
    # without one, each call allocates its own
    ops.trimul_forward(z, m, blob, "incoming")
    assert rec.of("kfh_trimul_forward")[-1][5] not in (None, ws.data_ptr())


def test_wrappers_refuse_inconsistent_arguments_before_any_call(rec):
    from kfold_amd import ops

    z = torch.zeros(1, 8, 8, 128, dtype=torch.bfloat16)
    m = torch.ones(1, 8, 8, dtype=torch.bool)
    blob = torch.zeros(16, dtype=torch.uint8)
    with pytest.raises(ValueError, match="direction"):
        ops.trimul_forward(z, m, blob, "sideways")
    with pytest.raises(ValueError, match=r"\[\*, N, N, C\]"):
        ops.trimul_forward(z[:, :4], m[:, :4], blob, "outgoing")
    with pytest.raises(ValueError, match="out must"):
        ops.trimul_forward(z, m, blob, "outgoing", out=torch.zeros(1, 8, 8, 128))
    with pytest.raises(ValueError, match="residual must"):
        ops.triattn_forward(z, m, blob, 4, True, residual=z.float())
    with pytest.raises(NotImplementedError):
        ops.trimul_forward(torch.zeros(1, 8, 8, 48, dtype=torch.bfloat16), m, blob, "outgoing")
    with pytest.raises(TypeError, match="bfloat16 and float32"):
        ops.trimul_forward(z.half(), m, blob, "outgoing")
    assert rec.names() == []
    # an empty batch returns without a call
    out = ops.trimul_forward(z[:0], m[:0], blob, "outgoing")
    assert out.shape == (0, 8, 8, 128) and rec.names() == []


def test_recurrent_trunk_call_sequence(rec):
    """lm_stack -> recurrence step with the input sum fused -> main_stack, once per recycle
    (reference: model/model.py:522-529)."""
    from kfold_amd import modules

    N = 8
    trunk = modules.ParcaeTrunk(128, lm_blocks=1, main_blocks=2).eval()
    z = torch.zeros(1, N, N, 128, dtype=torch.bfloat16)
    z_in = torch.zeros_like(z)
    z_lm = torch.zeros_like(z)
    pair = torch.ones(1, N, N, dtype=torch.bool)
    with torch.no_grad():
        out = trunk(z, z_in, z_lm, pair, num_recycles=1)
    assert out.data_ptr() == z.data_ptr()
    block = ["kfh_trimul_forward", "kfh_trimul_forward", "kfh_transition_forward"]
    recycle = block + ["kfh_parcae_step"] + block * 2
    assert rec.names() == recycle * 2
    for step in rec.of("kfh_parcae_step"):
        zp, u, u_add, blob, outp, rows, C, eps, io, stream = step
        assert zp == outp == z.data_ptr() and u_add == z_in.data_ptr()
        assert u not in (z.data_ptr(), z_lm.data_ptr(), z_in.data_ptr()), "the LM stack works on a copy"
        assert (rows, C, io) == (N * N, 128, 0)
    # the triangular block's transition has expansion 4 and no mask; the state stays in place
    tr = rec.of("kfh_transition_forward")
    assert all(c[9] == 4 and c[3] is None for c in tr)
    assert [c[0] == z.data_ptr() for c in tr] == [False, True, True] * 2
    assert len(rec.of("kfh_parcae_pack")) == 1 and len(rec.of("kfh_trimul_pack")) == 6


def test_serial_trunk_runs_blocks_in_order_on_the_same_tensors(rec):
    from kfold_amd import modules

    N = 8
    trunk = modules.PairformerTrunk(2, overlap_tracks=False).eval()
    z = torch.zeros(1, N, N, 128, dtype=torch.bfloat16)
    s = torch.zeros(1, N, 384, dtype=torch.bfloat16)
    tok = torch.ones(1, N, dtype=torch.bool)
    pair = tok[:, :, None] & tok[:, None, :]
    with torch.no_grad():
        z_out, s_out = trunk(z, s, pair, tok)
    assert z_out.data_ptr() == z.data_ptr() and s_out.data_ptr() == s.data_ptr()
    one = ["kfh_trimul_forward", "kfh_trimul_forward", "kfh_triattn_forward", "kfh_triattn_forward",
           "kfh_transition_forward", "kfh_pair_bias_project", "kfh_apb_forward", "kfh_transition_forward"]
    assert rec.names() == one * 2
    blobs = [c[2] for c in rec.of("kfh_trimul_forward")]
    assert len(set(blobs)) == 4, "each block's two tri-mul modules have their own packed weights"


def test_window_attention_flattens_leading_dimensions(rec):
    """[B, W, L, C] windows go to the library as B*W windows; the conditioned variant passes both
    conditioning tensors and the plain one none (reference:
    layers/folding/attention_pair_bias.py:206-260)."""
    from kfold_amd import layers

    B, W, Lq, Lk, C, H, Cs = 2, 3, 32, 128, 128, 4, 64
    a_q = torch.zeros(B, W, Lq, C, dtype=torch.bfloat16)
    a_k = torch.zeros(B, W, Lk, C, dtype=torch.bfloat16)
    bias = torch.zeros(B, W, H, Lq, Lk, dtype=torch.bfloat16)
    mask = torch.ones(B, W, Lk, dtype=torch.bool)
    with torch.no_grad():
        plain = layers.CrossAttentionPairBias(C, H, None).eval()
        out = plain(a_q, a_k, None, None, bias, mask)
        assert out.shape == a_q.shape and out.dtype == a_q.dtype
        cond = layers.CrossAttentionPairBias(C, H, Cs).eval()
        s_q = torch.zeros(B, W, Lq, Cs, dtype=torch.bfloat16)
        s_k = torch.zeros(B, W, Lk, Cs, dtype=torch.bfloat16)
        cond(a_q, a_k, s_q, s_k, bias, mask)
        with pytest.raises(AssertionError):
            cond(a_q, a_k, None, None, bias, mask)
    c0, c1 = rec.of("kfh_cross_apb_forward")
    assert c0[12:19] == (B * W, Lq, Lk, C, H, 0, 1) and c0[2] is None and c0[3] is None
    assert c1[12:19] == (B * W, Lq, Lk, C, H, Cs, 1) and c1[2] and c1[3]
    assert c0[8] is None, "the module's forward returns the update without a residual"
    assert c0[5] == 0, "bf16 pair bias is passed as it is"


def test_other_widths_take_the_generic_entry_points(rec):
    """Triangle multiplication at C=256 and triangle attention at C=64 (4 heads of 16) go through
    the same entry points; unsupported widths are refused by the size queries."""
    from kfold_amd import primitives

    m = torch.ones(2, 8, 8, dtype=torch.bool)
    with torch.no_grad():
        primitives.TriangleMultiplicationIncoming(256).eval()(torch.zeros(2, 8, 8, 256, dtype=torch.bfloat16), m)
        primitives.TriangleAttentionEndingNode(64, 4).eval()(torch.zeros(2, 8, 8, 64, dtype=torch.bfloat16), m)
        primitives.TriangleMultiplicationIncoming(64).eval()(torch.zeros(2, 8, 8, 64, dtype=torch.bfloat16), m)
        with pytest.raises(NotImplementedError):     # not a multiple of 32
            primitives.TriangleMultiplicationIncoming(48).eval()(torch.zeros(2, 8, 8, 48, dtype=torch.bfloat16), m)
    tm = rec.of("kfh_trimul_forward")[0]
    assert tm[7:11] == (2, 8, 256, 1)
    ta = rec.of("kfh_triattn_forward")[0]
    assert ta[7:12] == (2, 8, 64, 4, 1)


def test_pair_bias_attention_sharing_flags(rec):
    """Leading dimensions are flattened to samples; a bias, mask or conditioning tensor whose
    leading dimensions are all 1 is passed once and flagged as shared (reference shapes of the
    diffusion call site: a [B, S, L, C], s [B, S, L, Cs], bias [B, 1, H, L, L], mask [B, 1, L];
    layers/folding/attention_pair_bias.py:114-158)."""
    from kfold_amd import layers

    S, L, C, H, Cs = 5, 40, 768, 16, 384
    att = layers.SelfAttentionPairBias(C, H, Cs, "diffusion_global").eval()
    a = torch.zeros(1, S, L, C, dtype=torch.bfloat16)
    s = torch.zeros(1, S, L, Cs, dtype=torch.bfloat16)
    bias = torch.zeros(1, 1, H, L, L, dtype=torch.bfloat16)
    mask = torch.ones(1, 1, L, dtype=torch.bool)
    with torch.no_grad():
        out = att(a, s, bias, mask)
        assert out.shape == a.shape
        # per-sample bias and mask
        att(a, s, bias.expand(1, S, H, L, L), mask.expand(1, S, L))
        with pytest.raises(AssertionError):
            att(a, None, bias, mask)
    shared, per_sample = rec.of("kfh_apb_forward")
    # a, s_cond, tiles, mask, blob, residual, out, ws, ws_bytes, S, L, C, H, Cs, norm, bias/mask/s per sample
    assert shared[9:15] == (S, L, C, H, Cs, 1) and shared[15:18] == (0, 0, 1) and shared[1]
    assert per_sample[15:18] == (1, 1, 1)
    dense = rec.of("kfh_bias_tiles_from_dense")
    assert dense[0][3:6] == (1, H, L) and dense[1][3:6] == (S, H, L)
    # functional entry of the trunk call site: input already normalised, no conditioning, no norm
    plain = layers.SelfAttentionPairBias(384, 16, None, "confidence").eval()
    x = torch.zeros(2, L, 384, dtype=torch.bfloat16)
    with torch.no_grad():
        layers.hip_attention_pair_bias(plain, x, x, torch.zeros(2, 16, L, L, dtype=torch.bfloat16),
                                       torch.ones(2, L, dtype=torch.bool))
        # different tensors on the two sides: the cross entry, already normalised (apply_norm = 0)
        xk = torch.zeros(2, 2 * L, 384, dtype=torch.bfloat16)
        y = layers.hip_attention_pair_bias(plain, x, xk, torch.zeros(2, 16, L, 2 * L, dtype=torch.bfloat16),
                                           torch.ones(2, 2 * L, dtype=torch.bool))
        assert y.shape == x.shape
    fn = rec.of("kfh_apb_forward")[-1]
    assert fn[9:15] == (2, L, 384, 16, 0, 0) and fn[15:18] == (1, 1, 0) and fn[1] is None
    assert fn[20] == 0, "bf16 arithmetic for bf16 activations"
    cr = rec.of("kfh_cross_apb_forward")[-1]
    # ..., W, Lq, Lk, C, H, Cs, apply_norm, eps, io_dtype, arith
    assert cr[12:19] == (2, L, 2 * L, 384, 16, 0, 0) and cr[2] is None and cr[3] is None and cr[21] == 0


def test_fp32_arithmetic_is_selected_for_fp32_diffusion_calls(rec, monkeypatch):
    """The reference runs its diffusion stack in fp32 outside autocast (model/model.py:419): fp32
    activations at a diffusion call site select KFH_ARITH_F32 (blob, bias tiles, workspace and
    forward all made for it); the confidence call site, bf16 activations and autocast keep bf16."""
    from kfold_amd import layers

    L, C, H, Cs, S = 40, 256, 8, 128, 2
    att = layers.SelfAttentionPairBias(C, H, Cs, "diffusion_global").eval()
    a32 = torch.zeros(1, S, L, C)
    s32 = torch.zeros(1, S, L, Cs)
    bias = torch.zeros(1, 1, H, L, L)
    mask = torch.ones(1, 1, L, dtype=torch.bool)
    with torch.no_grad():
        att(a32, s32, bias, mask)
        att(a32.bfloat16(), s32.bfloat16(), bias, mask)
        with monkeypatch.context() as mp:          # autocast("cuda") cannot be entered without a GPU
            mp.setattr(torch, "is_autocast_enabled", lambda *a: True)
            att(a32, s32, bias, mask)
        att.arith = "bf16"
        att(a32, s32, bias, mask)
        conf = layers.SelfAttentionPairBias(C, H, None, "confidence").eval()
        conf(a32, None, bias, mask)
        win = layers.CrossAttentionPairBias(128, 4, None).eval()
        win(torch.zeros(3, 32, 128), torch.zeros(3, 128, 128), None, None, torch.zeros(3, 4, 32, 128),
            torch.ones(3, 128, dtype=torch.bool))
    fw = rec.of("kfh_apb_forward")
    assert [c[20] for c in fw] == [1, 0, 0, 0, 0]
    packs = rec.of("kfh_apb_pack")
    assert [c[18] for c in packs] == [1, 0, 0], "one blob per arithmetic, re-packed when it changes"
    tiles = rec.of("kfh_bias_tiles_from_dense")
    assert [c[6] for c in tiles] == [1, 0, 0, 0, 0]
    assert rec.of("kfh_cross_apb_forward")[-1][21] == 1 and rec.of("kfh_cross_apb_pack")[-1][24] == 1


def test_transition_rows_and_mask_plumbing(rec):
    from kfold_amd import layers

    tr = layers.Transition(128, 2).eval()
    tr.layernorm.eps = 2e-6
    x = torch.zeros(2, 6, 6, 128, dtype=torch.float32)
    with torch.no_grad():
        y = tr(x)
    assert y.shape == x.shape and y.dtype == x.dtype
    c = rec.of("kfh_transition_forward")[0]
    assert c[0] == x.data_ptr() and c[2] is None and c[3] is None and c[4] == y.data_ptr() != x.data_ptr()
    assert (c[7], c[8], c[9], c[11]) == (72, 128, 2, 1) and c[10] == pytest.approx(2e-6)
    assert c[5] is None and c[6] == 0, "the fused C=128 kernel needs no workspace"
    wide = layers.Transition(384, 4).eval()
    s = torch.zeros(3, 10, 384, dtype=torch.bfloat16)
    with torch.no_grad():
        wide(s)
    c = rec.of("kfh_transition_forward")[1]
    assert (c[7], c[8], c[9], c[11]) == (30, 384, 4, 0) and c[5] and c[6] > 0


def test_block_with_phases_over_row_ranges(rec):
    """phase_row_chunks = 2 at N = 300 (contraction tiles of 128 rows): every triangle op becomes one
    input phase over all rows, then core and output phase per range, in place on z; the transition
    and the default block are untouched."""
    from kfold_amd import _lib, modules

    N = 300
    blk = modules.PairformerBlock(phase_row_chunks=2).eval()
    z = torch.zeros(1, N, N, 128, dtype=torch.bfloat16)
    pair = torch.ones(1, N, N, dtype=torch.bool)
    waits = []
    with torch.no_grad():
        blk(z, pair, inplace_output=True, before_first_write=lambda: waits.append(len(rec.calls)))
    IN, CORE, OUT = _lib.KFH_STAGE_IN, _lib.KFH_STAGE_CORE, _lib.KFH_STAGE_OUT
    tm = rec.of("kfh_trimul_forward_rows")
    assert [(c[13], c[14], c[15]) for c in tm] == 2 * [(IN, 0, N), (CORE, 0, 128), (OUT, 0, 128),
                                                       (CORE, 128, 172), (OUT, 128, 172)]
    assert all(c[0] == c[3] == c[4] == z.data_ptr() and c[7] == 1 for c in tm)
    assert [c[10] for c in tm] == 5 * [0] + 5 * [1]                       # outgoing, then incoming
    ta = rec.of("kfh_triattn_forward_rows")
    assert [(c[14], c[15], c[16]) for c in ta] == 2 * [(IN, 0, N), (CORE, 0, 128), (OUT, 0, 128),
                                                       (CORE, 128, 172), (OUT, 128, 172)]
    assert [c[11] for c in ta] == 5 * [0] + 5 * [1]                       # starting, then ending node
    assert rec.names(("_forward", "_forward_stages")) == ["kfh_transition_forward"]
    # the caller's wait is placed after the input phase of the first op and before its first output phase
    first_in = next(i for i, (n, a) in enumerate(rec.calls) if n == "kfh_trimul_forward_rows")
    assert waits == [first_in + 1]
    # a range shorter than the attention kernel takes: the op runs in one piece
    rec.calls.clear()
    small = torch.zeros(1, 70, 70, 128, dtype=torch.bfloat16)
    with torch.no_grad():
        blk(small, torch.ones(1, 70, 70, dtype=torch.bool), inplace_output=True)
    assert rec.names(("_forward",)) == ["kfh_trimul_forward", "kfh_trimul_forward", "kfh_triattn_forward",
                                        "kfh_triattn_forward", "kfh_transition_forward"]


def test_phased_op_on_two_streams_orders_core_and_output(rec, monkeypatch):
    """The two-stream form of an op run in row ranges, with stand-ins for the streams and events: the
    input phase and every core phase are enqueued on the caller's stream, each output phase on the side
    stream after an event recorded behind its core phase, and the caller's stream waits for the side
    stream at the end."""
    from kfold_amd import _lib, ops

    log = []

    class FakeStream:
        def __init__(self, name):
            self.name, self.cuda_stream = name, 0

        def wait_event(self, ev):
            log.append((self.name, "wait_event", ev.id))

        def wait_stream(self, other):
            log.append((self.name, "wait_stream", other.name))

    class FakeEvent:
        count = 0

        def __init__(self):
            FakeEvent.count += 1
            self.id = FakeEvent.count

        def record(self, stream):
            log.append((stream.name, "record", self.id))

    main, side = FakeStream("main"), FakeStream("side")
    current = [main]

    class use_stream:
        def __init__(self, s):
            self.s = s

        def __enter__(self):
            self.prev, current[0] = current[0], self.s

        def __exit__(self, *a):
            current[0] = self.prev

    monkeypatch.setattr(torch.cuda, "current_stream", lambda dev=None: current[0])
    monkeypatch.setattr(torch.cuda, "Event", FakeEvent)
    monkeypatch.setattr(torch.cuda, "stream", use_stream)
    monkeypatch.setattr(ops, "_stream", lambda dev: log.append((current[0].name, "launch")) or 0)

    N = 300
    z = torch.zeros(1, N, N, 128, dtype=torch.bfloat16)
    blob = torch.zeros(_lib.lib().kfh_trimul_packed_bytes(128), dtype=torch.uint8)
    waits = []
    ops.trimul_forward(z, torch.ones(1, N, N, dtype=torch.bool), blob, "outgoing", residual=z, out=z,
                       row_chunks=3, side=side, before_write=lambda: waits.append(len(log)))
    IN, CORE, OUT = _lib.KFH_STAGE_IN, _lib.KFH_STAGE_CORE, _lib.KFH_STAGE_OUT
    calls = [(c[13], c[14], c[15]) for c in rec.of("kfh_trimul_forward_rows")]
    assert calls == [(IN, 0, N), (CORE, 0, 128), (OUT, 0, 128), (CORE, 128, 128), (OUT, 128, 128),
                     (CORE, 256, 44), (OUT, 256, 44)]
    assert log == [("main", "launch"),                                             # input phase
                   ("main", "launch"), ("main", "record", 1), ("side", "wait_event", 1), ("side", "launch"),
                   ("main", "launch"), ("main", "record", 2), ("side", "wait_event", 2), ("side", "launch"),
                   ("main", "launch"), ("main", "record", 3), ("side", "wait_event", 3), ("side", "launch"),
                   ("main", "wait_stream", "side")]
    assert waits == [1], "the caller's wait comes right after the input phase, before anything is written"
