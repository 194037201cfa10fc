"""Random shapes, masks, dtypes and call options of every operator, run on the kernels' host build
and compared with the oracle.

TEST INFRASTRUCTURE.  ``python -m tests.hostsim.fuzz [--seeds A:B] [--family NAME]`` draws one case
per seed (the seed fixes family, shape and data, so a failing case is re-run by its seed), runs
module -> functional layer -> C ABI -> kernel code on the host build and checks the result against
the oracle at the tolerances of the parity tests.  ``tests/test_hostsim_fuzz.py`` runs a fixed small
range of seeds in the CPU suite.
"""

from __future__ import annotations

import argparse
import random
import sys
import time
import traceback

import torch

from kfold_amd import synthetic
from tests import hostsim
from tests.util import assert_close

F32_ARITH_MAX_ABS = 1e-4
BIG = False          # --big: sizes up to a few hundred tokens (seconds to a minute per case)


def _affine(module, g):
    with torch.no_grad():
        for name, p in module.named_parameters():
            if p.dim() == 1:
                if name.endswith("bias"):
                    p.copy_(0.1 * torch.randn(p.shape, generator=g))
                else:
                    p.copy_(1 + 0.2 * torch.randn(p.shape, generator=g))


def _pair(ref_cls, hip_cls, args, seed, std, g, dev):
    ref = ref_cls(*args).eval()
    synthetic.init_weights_(ref, seed, std=std)
    _affine(ref, g)
    hip = hip_cls(*args).eval()
    hip.load_state_dict(ref.state_dict())
    return ref, hip.to(dev)


def _size(r: random.Random, hi: int) -> int:
    """A size in 1..hi, half of the time right at a multiple of 32 or next to one (where tiles,
    key blocks and padded planes begin and end)."""
    if r.random() < 0.5:
        edges = [v for m in range(0, hi + 32, 32) for v in (m - 1, m, m + 1) if 1 <= v <= hi]
        return r.choice(edges)
    return r.randint(1, hi)


def _pair_mask(r: random.Random, g, batch: int, n: int) -> torch.Tensor:
    kind = r.choice(["tokens", "random", "sparse", "full", "rows_off", "one_key"])
    if kind == "tokens":
        ms = [synthetic.pair_mask_from_tokens(synthetic.token_mask(n, r.randint(0, max(0, n - 1))))[0] for _ in range(batch)]
        m = torch.stack(ms)
    elif kind == "random":
        m = torch.rand(batch, n, n, generator=g) > 0.3
    elif kind == "sparse":
        m = torch.rand(batch, n, n, generator=g) > 0.9
    elif kind == "full":
        m = torch.ones(batch, n, n, dtype=torch.bool)
    elif kind == "rows_off":
        m = torch.rand(batch, n, n, generator=g) > 0.2
        m[:, r.randrange(n), :] = False
        m[:, :, r.randrange(n)] = False
    else:
        m = torch.zeros(batch, n, n, dtype=torch.bool)
        m[:, :, r.randrange(n)] = True
    return m


def case_trimul(r, g, dev):
    from kfold_amd import ops, primitives as P
    from oracle import torch_path as O

    c = r.choice([128, 128, 256, 64, 64, 32, 96, 160])
    n = _size(r, 70 if c == 256 else 110) if not BIG else _size(r, 160 if c == 256 else 280)
    batch = r.choice([1, 1, 2, 3])
    incoming = r.random() < 0.5
    dtype = r.choice([torch.bfloat16, torch.bfloat16, torch.float32])
    cls = "TriangleMultiplicationIncoming" if incoming else "TriangleMultiplicationOutgoing"
    what = f"trimul C={c} N={n} B={batch} {cls[22:]} {dtype}"
    ref, hip = _pair(getattr(O, cls), getattr(P, cls), (c,), r.randrange(100), 0.02 * 128 / c if c < 128 else 0.02, g, dev)
    x = torch.randn(batch, n, n, c, generator=g).to(dtype)
    mask = _pair_mask(r, g, batch, n)
    with torch.no_grad():
        want = ref(x.float(), mask)
        xd, md = x.to(dev), mask.to(dev)
        got = hip(xd, md)
        assert got.dtype == dtype and got.shape == x.shape, what
        e = assert_close(got, want, what, auto_scale=True)
        if r.random() < 0.5:
            direction = "incoming" if incoming else "outgoing"
            xin = xd.clone()
            ops.trimul_forward(xin, md, hip._hip_multiplication_cache, direction, residual=xin, out=xin)
            assert_close(xin, x.float() + want, what + " residual in place", rel_fro=5e-3, auto_scale=True)
    return what, e


def case_triattn(r, g, dev):
    from kfold_amd import ops, primitives as P
    from oracle import torch_path as O

    c, h = r.choice([(128, 4), (128, 4), (64, 4), (64, 4), (96, 2), (32, 2), (64, 1), (128, 8), (64, 2), (160, 5)])
    n = _size(r, 100) if not BIG else _size(r, 200)
    batch = r.choice([1, 1, 2, 4]) if not BIG else r.choice([1, 1, 2])
    starting = r.random() < 0.5
    dtype = r.choice([torch.bfloat16, torch.bfloat16, torch.float32])
    cls = "TriangleAttentionStartingNode" if starting else "TriangleAttentionEndingNode"
    what = f"triattn C={c} H={h} N={n} B={batch} {cls[17:]} {dtype}"
    ref, hip = _pair(getattr(O, cls), getattr(P, cls), (c, h), r.randrange(100), r.choice([0.02, 0.08]), g, dev)
    x = torch.randn(batch, n, n, c, generator=g).to(dtype)
    mask = None if r.random() < 0.15 else _pair_mask(r, g, batch, n)
    with torch.no_grad():
        want = torch.stack([ref(x[b:b + 1].float(), None if mask is None else mask[b:b + 1].float())[0]
                            for b in range(batch)])
        xd = x.to(dev)
        md = None if mask is None else mask.to(dev)
        got = hip(xd, md)
        assert got.dtype == dtype and got.shape == x.shape, what
        e = assert_close(got, want, what, auto_scale=True)
        if r.random() < 0.5:
            xin = xd.clone()
            ops.triattn_forward(xin, md, hip._hip_attention_cache, h, starting, residual=xin, out=xin)
            assert_close(xin, x.float() + want, what + " residual in place", rel_fro=5e-3, auto_scale=True)
    return what, e


def case_transition(r, g, dev):
    from kfold_amd.layers import Transition, hip_transition
    from oracle import torch_path as O

    c = r.choice([128, 128, 256, 384, 768, 64, 32, 96, 160])
    e_ = r.choice([2, 4, 2, 4, 1, 3])
    rows = _size(r, 1500 if c <= 256 else 300)
    dtype = r.choice([torch.bfloat16, torch.float32])
    what = f"transition C={c} E={e_} rows={rows} {dtype}"
    ref, hip = _pair(O.Transition, Transition, (c, e_), r.randrange(100), 0.05, g, dev)
    x = torch.randn(rows, c, generator=g).to(dtype)
    with torch.no_grad():
        want = ref(x.float())
        got = hip(x.to(dev))
        assert got.dtype == dtype, what
        e = assert_close(got, want, what, auto_scale=True)
        xin = x.to(dev).clone()
        if r.random() < 0.5:
            mask = torch.rand(rows, generator=g) > 0.3
            hip_transition(hip, xin, residual=xin, mask=mask.to(dev), out=xin)
            want2 = (x.float() + want) * mask[:, None]
            assert (xin.cpu()[~mask] == 0).all(), what
        else:
            hip_transition(hip, xin, residual=xin, out=xin)
            want2 = x.float() + want
        assert_close(xin, want2, what + " residual", rel_fro=5e-3, auto_scale=True)
    return what, e


def case_apb(r, g, dev):
    from kfold_amd.layers import SelfAttentionPairBias
    from oracle import torch_path as O

    diffusion = r.random() < 0.6
    L = _size(r, 150) if not BIG else _size(r, 400)
    S = r.randint(1, 4) if diffusion else 1
    dtype = r.choice([torch.bfloat16, torch.float32])
    args = (768, 16, 384, "diffusion_global") if diffusion else (384, 16, None, "confidence")
    ref, hip = _pair(O.SelfAttentionPairBias, SelfAttentionPairBias, args, r.randrange(100), 0.03, g, dev)
    ca = args[0]
    a = torch.randn(1, S, L, ca, generator=g).to(dtype)
    s_shared = r.random() < 0.5
    s = torch.randn(1, 1 if s_shared else S, L, 384, generator=g).to(dtype) if diffusion else None
    bias = torch.randn(1, 1, 16, L, L, generator=g)
    mask = torch.rand(1, 1, L, generator=g) > r.choice([0.0, 0.15, 0.6])
    if r.random() < 0.1:
        mask[:] = False
    f32_arith = diffusion and dtype == torch.float32
    what = f"apb {'diffusion' if diffusion else 'confidence'} L={L} S={S} {dtype} s_shared={s_shared}"
    with torch.no_grad():
        if diffusion:
            want = ref(a.float(), s.float().expand(1, S, L, 384), bias, mask)
            got = hip(a.to(dev), s.to(dev), bias.to(dev), mask.to(dev))
        else:
            want = ref(a.float(), None, bias, mask)
            got = hip(a.to(dev), None, bias.to(dev), mask.to(dev))
    assert got.shape == a.shape and got.dtype == dtype, what
    if f32_arith:
        e = assert_close(got, want, what + " (fp32 arithmetic)", max_abs=F32_ARITH_MAX_ABS, mean_abs=1e-5, rel_fro=1e-5)
    else:
        e = assert_close(got, want, what, auto_scale=True)
    return what, e


def case_cross(r, g, dev):
    from kfold_amd.layers import CrossAttentionPairBias
    from oracle import torch_path as O

    cond = r.random() < 0.5
    S, W = r.randint(1, 3), r.randint(1, 7)
    Lq, Lk = r.choice([32, 32, r.randint(1, 40)]), r.choice([128, 128, r.randint(1, 140)])
    dtype = r.choice([torch.bfloat16, torch.float32])
    what = f"cross windows S={S} W={W} {Lq}x{Lk} cond={cond} {dtype}"
    ref, hip = _pair(O.CrossAttentionPairBias, CrossAttentionPairBias, (128, 4, 128 if cond else None),
                     r.randrange(100), 0.05, g, dev)
    mk = lambda n: torch.randn(S, W, n, 128, generator=g).to(dtype)
    aq, ak = mk(Lq), mk(Lk)
    sq, sk = (mk(Lq), mk(Lk)) if cond else (None, None)
    bias = torch.randn(1, W, 4, Lq, Lk, generator=g)
    mask = torch.rand(1, W, Lk, generator=g) > r.choice([0.0, 0.2, 0.7])
    if W > 1 and r.random() < 0.3:
        mask[0, r.randrange(W)] = False
    f = lambda t: None if t is None else t.float()
    d = lambda t: None if t is None else t.to(dev)
    with torch.no_grad():
        want = ref(aq.float(), ak.float(), f(sq), f(sk), bias, mask)
        got = hip(d(aq), d(ak), d(sq), d(sk), bias.to(dev), mask.to(dev))
    assert got.shape == aq.shape and got.dtype == dtype, what
    if dtype == torch.float32:
        e = assert_close(got, want, what + " (fp32 arithmetic)", max_abs=F32_ARITH_MAX_ABS, mean_abs=1e-5, rel_fro=1e-5)
    else:
        e = assert_close(got, want, what, auto_scale=True)
    return what, e


def case_parcae(r, g, dev):
    from kfold_amd import modules as M
    from oracle import torch_path as O

    C = r.choice([128, 256])
    rows_shape = r.choice([(1, r.randint(1, 40)), (r.randint(1, 3), r.randint(1, 25))])
    dtype = r.choice([torch.bfloat16, torch.float32])
    what = f"parcae C={C} B={rows_shape[0]} N={rows_shape[1]} {dtype}"
    ref = O.ParcaeStep(C).eval()
    with torch.no_grad():
        ref.parcae_log_a.copy_(0.3 * torch.randn(C, generator=g))
        ref.parcae_log_delta.add_(0.5 * torch.randn(C, generator=g))
        ref.parcae_b_cont.add_(0.05 * torch.randn(C, C, generator=g))
        ref.layernorm_z.weight.copy_(1 + 0.2 * torch.randn(C, generator=g))
        ref.layernorm_z.bias.copy_(0.1 * torch.randn(C, generator=g))
    hip = M.ParcaeStep(C).eval()
    hip.load_state_dict(ref.state_dict())
    hip.to(dev)
    b, n = rows_shape
    z = torch.randn(b, n, n, C, generator=g).to(dtype)
    u = (2.0 * torch.randn(b, n, n, C, generator=g) + 0.5).to(dtype)
    with torch.no_grad():
        want = ref(z.float(), u.float())
        got = hip(z.to(dev), u.to(dev), inplace=False)
    e = assert_close(got, want, what, rel_fro=5e-3)
    return what, e


def case_block(r, g, dev):
    """One PairSingleBlock update by update (each in-place update against the oracle op on the very
    same input), the way the block tests do at the quoted sizes."""
    from kfold_amd import modules as M
    from oracle import torch_path as O

    n = _size(r, 72) if not BIG else _size(r, 200)
    n_pad = r.randint(0, max(0, n - 1))
    what = f"pair+single block N={n} pad={n_pad}"
    ref = O.PairSingleBlock().eval()
    synthetic.init_weights_(ref, r.randrange(100), std=r.choice([0.02, 0.05]))
    _affine(ref, g)
    hip = M.PairSingleBlock().eval()
    hip.load_state_dict(ref.state_dict())
    hip.to(dev)
    z, tok, pm = synthetic.pair_inputs(n, 128, n_pad, seed=r.randrange(1000))
    s = synthetic.single_inputs(n, 384, seed=r.randrange(1000))
    with torch.no_grad():
        zw, sw = ref(z.bfloat16().float(), s.bfloat16().float(), pm, tok)
        zg, sg = hip(z.bfloat16().to(dev), s.bfloat16().to(dev), pm.to(dev), tok.to(dev))
    # a bf16 residual stream of O(1..5) values: the absolute limits scale with the stream
    e = assert_close(zg, zw, what + " z", auto_scale=True, max_abs=6e-2, mean_abs=4e-3)
    assert_close(sg, sw, what + " s", auto_scale=True, max_abs=6e-2, mean_abs=4e-3)
    assert (zg.float().cpu()[~pm.expand_as(zg[..., 0])] == 0).all(), what + ": masked positions not zero"
    return what, e


def case_wide_block(r, g, dev):
    """The shipping trunk's TriangularBlock at c_z = 256 (tri-mul out, in, transition x4), fp32 stream."""
    from kfold_amd import modules as M
    from oracle import torch_path as O

    n = _size(r, 70) if not BIG else _size(r, 140)
    n_pad = r.randint(0, max(0, n - 1))
    what = f"triangular block C=256 N={n} pad={n_pad}"
    ref = O.TriangularBlock(256).eval()
    synthetic.init_weights_(ref, r.randrange(100))
    _affine(ref, g)
    hip = M.TriangularBlock(256).eval()
    hip.load_state_dict(ref.state_dict())
    hip.to(dev)
    z, _, pm = synthetic.pair_inputs(n, 256, n_pad, seed=r.randrange(1000))
    with torch.no_grad():
        zw = ref(z.clone(), pm.float())
        zin = z.clone().to(dev)
        zg = hip(zin, pm.to(dev))
    assert zg.data_ptr() == zin.data_ptr(), what
    e = assert_close(zg, zw, what, rel_fro=5e-3, auto_scale=True)
    return what, e


def case_template_block(r, g, dev):
    """The apo template stack's whole Pairformer block at c_z = 64 over a batch of templates, in
    place with the final mask, fp32 stream."""
    from kfold_amd import modules as M
    from oracle import torch_path as O

    n = _size(r, 64) if not BIG else _size(r, 130)
    batch = r.randint(1, 4)
    what = f"template block C=64 N={n} B={batch}"
    ref = O.PairformerBlock(64, 4).eval()
    synthetic.init_weights_(ref, r.randrange(100), std=0.05)
    _affine(ref, g)
    hip = M.PairformerBlock(64, 4).eval()
    hip.load_state_dict(ref.state_dict())
    hip.to(dev)
    z = torch.randn(batch, n, n, 64, generator=g)
    pm = torch.stack([synthetic.pair_mask_from_tokens(synthetic.token_mask(n, r.randint(0, max(0, n - 1))))[0]
                      for _ in range(batch)])
    with torch.no_grad():
        zw = torch.stack([ref(z[b:b + 1].clone(), pm[b:b + 1].float())[0] for b in range(batch)])
        zin = z.clone().to(dev)
        zg = hip(zin, pm.to(dev), inplace_output=True)
    assert zg.data_ptr() == zin.data_ptr(), what
    e = assert_close(zg, zw, what, rel_fro=5e-3, auto_scale=True)
    assert (zg.cpu()[~pm] == 0).all(), what + ": masked positions not zero"
    return what, e


def _dirty_workspace(arena, nbytes: int, g) -> torch.Tensor:
    """A caller-owned workspace (256-byte aligned) full of random bytes."""
    ws = arena.bytes(max(nbytes, 256), 256)
    ws.copy_(torch.randint(0, 256, (ws.numel(),), generator=g, dtype=torch.uint8))
    return ws


def case_api(r, g, dev, arena=None):
    """Call options that must not change a single bit: a caller-owned (dirty) workspace, the split
    into stages with a callback before the first write, masks given as float / uint8 / broadcastable
    tensors, non-contiguous activations, the batched and the per-element workspace of a template
    batch, and the allocation-free transition entry against the workspace-taking one."""
    from kfold_amd import _lib, ops, primitives as P
    from kfold_amd.layers import Transition
    from kfold_amd.layers.transition import _parameters

    kind = r.choice(["trimul", "triattn", "transition_static"])
    if kind == "trimul":
        c = r.choice([128, 256, 64, 96])
        n = _size(r, 60 if c == 256 else 90)
        batch = r.choice([1, 1, 2, 3])
        incoming = r.random() < 0.5
        what = f"api trimul C={c} N={n} B={batch} incoming={incoming}"
        cls = "TriangleMultiplicationIncoming" if incoming else "TriangleMultiplicationOutgoing"
        hip = getattr(P, cls)(c).eval()
        synthetic.init_weights_(hip, r.randrange(100), std=0.05)
        _affine(hip, g)
        hip.to(dev)
        x = torch.randn(batch, n, n, c, generator=g).bfloat16().to(dev)
        mask = _pair_mask(r, g, batch, n).to(dev)
        direction = "incoming" if incoming else "outgoing"
        with torch.no_grad():
            base = hip(x, mask)
            blob = hip._hip_multiplication_cache
            ws = _dirty_workspace(arena, ops.workspace_bytes("trimul", N=n, C=c), g)
            assert torch.equal(ops.trimul_forward(x, mask, blob, direction, workspace=ws), base), what + ": workspace"
            if batch > 1:
                wsb = _dirty_workspace(arena, ops.workspace_bytes("trimul", N=n, C=c, B=batch), g)
                assert torch.equal(ops.trimul_forward(x, mask, blob, direction, workspace=wsb), base), what + ": batched workspace"
            calls = []
            assert torch.equal(ops.trimul_forward(x, mask, blob, direction, before_write=lambda: calls.append(1)), base), what + ": stages"
            assert calls == [1], what
            assert torch.equal(ops.trimul_forward(x, mask.float(), blob, direction), base), what + ": float mask"
            assert torch.equal(ops.trimul_forward(x, mask.to(torch.uint8) * 3, blob, direction), base), what + ": uint8 mask"
            xt = x.transpose(1, 2).contiguous().transpose(1, 2)          # same values, other strides
            assert not xt.is_contiguous() or n == 1
            assert torch.equal(ops.trimul_forward(xt, mask, blob, direction), base), what + ": strided input"
            out = x.clone()
            ops.trimul_forward(out, mask, blob, direction, residual=out, out=out, before_write=lambda: None)
            want = x.clone()
            ops.trimul_forward(x, mask, blob, direction, residual=x.clone(), out=want)
            assert torch.equal(out, want), what + ": in place with stages"
        return what, {"max_abs": 0.0, "rel_fro": 0.0}
    if kind == "triattn":
        c, h = r.choice([(128, 4), (64, 4), (96, 2)])
        n = _size(r, 70)
        batch = r.choice([1, 2, 4])
        starting = r.random() < 0.5
        what = f"api triattn C={c} H={h} N={n} B={batch} starting={starting}"
        cls = "TriangleAttentionStartingNode" if starting else "TriangleAttentionEndingNode"
        hip = getattr(P, cls)(c, h).eval()
        synthetic.init_weights_(hip, r.randrange(100), std=0.08)
        _affine(hip, g)
        hip.to(dev)
        x = torch.randn(batch, n, n, c, generator=g).bfloat16().to(dev)
        mask = _pair_mask(r, g, batch, n).to(dev)
        with torch.no_grad():
            base = hip(x, mask)
            blob = hip._hip_attention_cache
            ws = _dirty_workspace(arena, ops.workspace_bytes("triattn", N=n, C=c, heads=h), g)
            assert torch.equal(ops.triattn_forward(x, mask, blob, h, starting, workspace=ws), base), what + ": workspace"
            if batch > 1:
                wsb = _dirty_workspace(arena, ops.workspace_bytes("triattn", N=n, C=c, heads=h, B=batch), g)
                assert torch.equal(ops.triattn_forward(x, mask, blob, h, starting, workspace=wsb), base), what + ": batched workspace"
            assert torch.equal(ops.triattn_forward(x, mask.float(), blob, h, starting), base), what + ": float mask"
            ones = torch.ones(batch, n, n, dtype=torch.bool).to(dev)
            assert torch.equal(ops.triattn_forward(x, None, blob, h, starting),
                               ops.triattn_forward(x, ones, blob, h, starting)), what + ": mask=None vs all ones"
            xt = x.transpose(1, 2).contiguous().transpose(1, 2)
            assert torch.equal(ops.triattn_forward(xt, mask, blob, h, starting), base), what + ": strided input"
        return what, {"max_abs": 0.0, "rel_fro": 0.0}
    # the allocation-free transition entry: same bits as the workspace-taking one, on calls in a row
    C, E = r.choice([(384, 4), (768, 2), (128, 2), (256, 4), (64, 4), (96, 3)])
    mod = Transition(C, E).eval()
    synthetic.init_weights_(mod, r.randrange(100), std=0.05)
    mod.to(dev)
    blob = ops.transition_pack(*_parameters(mod), device=dev)
    L = _lib.lib()
    what = f"api static transition C={C} E={E}"
    for _ in range(3):
        rows = _size(r, 600)
        dtype = r.choice([torch.bfloat16, torch.float32])
        residual = r.random() < 0.5
        x = torch.randn(rows, C, generator=g).to(dtype).to(dev)
        io = _lib.KFH_BF16 if dtype == torch.bfloat16 else _lib.KFH_F32
        res = x.clone() if residual else None
        want = ops.transition_forward(x, blob, E, residual=res)
        got = torch.full_like(x, float("nan"))
        need = L.kfh_transition_workspace_bytes(rows, C, E)
        rc = L.kfh_transition_forward_static(x.data_ptr(), blob.data_ptr(), None if res is None else res.data_ptr(),
                                             None, got.data_ptr(), rows, C, E, 1e-5, io, None)
        if need > L.kfh_transition_static_scratch_bytes():
            assert rc != 0, what + f": rows={rows} beyond the static scratch was accepted"
            continue
        _lib.check(rc)
        assert torch.equal(got, want), what + f": rows={rows} {dtype} residual={residual}"
    return what, {"max_abs": 0.0, "rel_fro": 0.0}


def case_ranges(r, g, dev):
    """Core and output phase over ranges of rows against the op in one piece: same bits, for random
    sizes (not multiples of the tiles), range counts, directions / nodes, dtypes, in place or not."""
    from kfold_amd import ops, primitives as P

    dtype = r.choice([torch.bfloat16, torch.float32])
    inplace = r.random() < 0.5
    if r.random() < 0.5:
        c = r.choice([128, 256])
        n = r.randint(257, 384)                     # planes of 384 rows: three tile rows of 128
        incoming = r.random() < 0.5
        chunks = r.randint(2, 4)
        what = f"ranges trimul C={c} N={n} incoming={incoming} chunks={chunks} {dtype} inplace={inplace}"
        cls = "TriangleMultiplicationIncoming" if incoming else "TriangleMultiplicationOutgoing"
        mod = synthetic.init_weights_(getattr(P, cls)(c).eval(), r.randrange(100), std=0.05).to(dev)
        x = torch.randn(1, n, n, c, generator=g).to(dtype).to(dev)
        mask = _pair_mask(r, g, 1, n).to(dev)
        with torch.no_grad():
            mod(x[:, :4, :4].contiguous(), mask[:, :4, :4].contiguous())
            blob, d = mod._hip_multiplication_cache, mod.direction
            if inplace:
                a, b = x.clone(), x.clone()
                ops.trimul_forward(a, mask, blob, d, residual=a, out=a)
                ops.trimul_forward(b, mask, blob, d, residual=b, out=b, row_chunks=chunks)
            else:
                a = ops.trimul_forward(x, mask, blob, d)
                b = ops.trimul_forward(x, mask, blob, d, row_chunks=chunks)
        assert torch.equal(a, b), what
        return what, {"max_abs": 0.0, "rel_fro": 0.0}
    n = r.randint(129, 300)
    starting = r.random() < 0.5
    chunks = r.randint(2, 4)
    what = f"ranges triattn N={n} starting={starting} chunks={chunks} {dtype} inplace={inplace}"
    cls = "TriangleAttentionStartingNode" if starting else "TriangleAttentionEndingNode"
    mod = synthetic.init_weights_(getattr(P, cls)(128, 4).eval(), r.randrange(100), std=0.08).to(dev)
    x = torch.randn(1, n, n, 128, generator=g).to(dtype).to(dev)
    mask = _pair_mask(r, g, 1, n).to(dev)
    with torch.no_grad():
        mod(x[:, :4, :4].contiguous(), mask[:, :4, :4].contiguous())
        blob = mod._hip_attention_cache
        if inplace:
            a, b = x.clone(), x.clone()
            ops.triattn_forward(a, mask, blob, 4, starting, residual=a, out=a)
            ops.triattn_forward(b, mask, blob, 4, starting, residual=b, out=b, row_chunks=chunks)
        else:
            a = ops.triattn_forward(x, mask, blob, 4, starting)
            b = ops.triattn_forward(x, mask, blob, 4, starting, row_chunks=chunks)
    assert torch.equal(a, b), what
    return what, {"max_abs": 0.0, "rel_fro": 0.0}


FAMILIES = {
    "trimul": case_trimul, "triattn": case_triattn, "transition": case_transition, "apb": case_apb,
    "cross": case_cross, "parcae": case_parcae, "block": case_block,
    "wide_block": case_wide_block, "template_block": case_template_block, "api": case_api,
    "ranges": case_ranges,
}
_ORDER = ["trimul", "triattn", "transition", "apb", "cross", "parcae", "block", "trimul", "triattn", "apb"]


def run_seed(seed: int, family: str | None = None):
    """(description, errors) of the case of this seed; raises on a mismatch."""
    r = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    fam = family or _ORDER[seed % len(_ORDER)]
    with hostsim.host_backend() as arena:
        if fam == "api":
            return case_api(r, g, hostsim.HostDevice("cpu"), arena)
        return FAMILIES[fam](r, g, hostsim.HostDevice("cpu"))


def main(argv: list[str]) -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--seeds", default="0:50", help="A:B = seeds A..B-1")
    ap.add_argument("--family", choices=sorted(FAMILIES), default=None)
    ap.add_argument("--big", action="store_true", help="larger sizes (another case per seed than without)")
    args = ap.parse_args(argv)
    global BIG
    BIG = args.big
    lo, hi = (int(v) for v in args.seeds.split(":"))
    failed = []
    for seed in range(lo, hi):
        t0 = time.time()
        try:
            what, e = run_seed(seed, args.family)
            print(f"seed {seed}: ok   {what}  max_abs {e['max_abs']:.2e} rel_fro {e['rel_fro']:.2e}  ({time.time() - t0:.1f} s)",
                  flush=True)
        except Exception as exc:  # noqa: BLE001 (every failure is reported with its seed)
            failed.append(seed)
            print(f"seed {seed}: FAIL {type(exc).__name__}: {str(exc)[:600]}", flush=True)
            traceback.print_exc(limit=3)
    print(f"{hi - lo - len(failed)} of {hi - lo} seeds passed; failed: {failed}", flush=True)
    return 1 if failed else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
