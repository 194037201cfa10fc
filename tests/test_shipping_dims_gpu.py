"""The pair widths the shipping model uses (configs/kfold.yaml of the reference): triangle
multiplication and the trunk's TriangularBlock at c_z = 256 (model/modules/tri_stack.py:119-125),
triangle attention at c = 64 with 4 heads of 16 batched over templates
(model/modules/apo_module.py:376-384)."""

import pytest
import torch

from kfold_amd import synthetic
from tests.util import assert_close

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _affine(ref, seed=77):
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for name, p in ref.named_parameters():
            if p.dim() == 1:
                if name.endswith("bias"):
                    p.copy_(0.1 * torch.randn(p.shape, generator=g))
                else:
                    p.copy_(1 + 0.2 * torch.randn(p.shape, generator=g))


@pytest.mark.parametrize("direction", ["outgoing", "incoming"])
@pytest.mark.parametrize("n,n_pad,dtype", [(70, 9, torch.bfloat16), (130, 0, torch.bfloat16), (33, 4, torch.float32)])
def test_trimul_c256(direction, n, n_pad, dtype):
    from kfold_amd import ops, primitives as P
    from oracle import torch_path as O

    print(f"case trimul C=256 {direction} n={n} {dtype}", flush=True)
    cls = "TriangleMultiplicationOutgoing" if direction == "outgoing" else "TriangleMultiplicationIncoming"
    ref = getattr(O, cls)(256).eval()
    synthetic.init_weights_(ref, 3)
    _affine(ref)
    hip = getattr(P, cls)(256).eval()
    hip.load_state_dict(ref.state_dict())
    hip.to(DEV)
    z, _, pm = synthetic.pair_inputs(n, 256, n_pad, seed=n)
    if n == 130:        # a general (not outer-product) mask
        pm = torch.rand(1, n, n, generator=torch.Generator().manual_seed(5)) > 0.3
    zi = z.to(dtype)
    with torch.no_grad():
        want = ref(zi.float(), pm)
        zd, pmd = zi.to(DEV), pm.to(DEV)
        got = hip(zd, pmd)
        assert got.dtype == dtype
        print(assert_close(got, want, f"trimul C=256 {direction}"), flush=True)
        assert torch.equal(got, hip(zd, pmd)), "run-to-run results differ"
        # fused residual in place
        zin = zd.clone()
        ops.trimul_forward(zin, pmd, hip._hip_multiplication_cache, direction, residual=zin, out=zin)
        assert_close(zin, zi.float() + want, "trimul C=256 residual in place", rel_fro=5e-3)


def test_triangular_block_c256():
    """The shipping trunk block: tri-mul out, tri-mul in, transition x4 at c_z = 256, in place."""
    from kfold_amd import modules as M
    from oracle import torch_path as O

    print("case triangular block C=256", flush=True)
    ref = O.TriangularBlock(256).eval()
    synthetic.init_weights_(ref, 11)
    hip = M.TriangularBlock(256).eval()
    hip.load_state_dict(ref.state_dict())
    hip.to(DEV)
    n = 80
    z, _, pm = synthetic.pair_inputs(n, 256, 10, seed=12)
    zb = z.bfloat16()
    with torch.no_grad():
        zw = ref(zb.float(), pm.float())
        zin = zb.float().to(DEV)
        zg = hip(zin, pm.to(DEV))
        assert zg.data_ptr() == zin.data_ptr()
        print(assert_close(zg, zw, "triangular block C=256 (fp32 stream)", rel_fro=5e-3), flush=True)
        zg16 = hip(zb.to(DEV), pm.to(DEV))
        # bf16 stream: three storage roundings of |z| up to ~5 on top of the kernel error
        print(assert_close(zg16, zw, "triangular block C=256 (bf16 stream)", max_abs=6e-2, mean_abs=4e-3,
                           rel_fro=5e-3), flush=True)


@pytest.mark.parametrize("starting", [True, False])
@pytest.mark.parametrize("c,h,n,batch", [(64, 4, 50, 4), (64, 4, 128, 1), (96, 2, 37, 2)])
def test_triattn_other_widths_batched(starting, c, h, n, batch):
    """c = 64, 4 heads x 16 with a leading batch of 4 (the apo stack's shape); 2 heads x 48 covers
    the 64-wide padded head."""
    from kfold_amd import ops, primitives as P
    from oracle import torch_path as O

    print(f"case triattn c={c} h={h} n={n} batch={batch} starting={starting}", flush=True)
    cls = "TriangleAttentionStartingNode" if starting else "TriangleAttentionEndingNode"
    ref = getattr(O, cls)(c, h).eval()
    synthetic.init_weights_(ref, 13, std=0.08)
    _affine(ref)
    hip = getattr(P, cls)(c, h).eval()
    hip.load_state_dict(ref.state_dict())
    hip.to(DEV)
    g = torch.Generator().manual_seed(n)
    x = torch.randn(batch, n, n, c, generator=g).bfloat16()
    mask = torch.rand(batch, n, n, generator=g) > 0.25
    mask[0, 3, :] = False                 # a fully masked row / column
    mask[0, :, 5] = False
    if batch > 1:
        mask[1] = synthetic.pair_mask_from_tokens(synthetic.token_mask(n, 7))[0]
    with torch.no_grad():
        want = torch.stack([ref(x[b:b + 1].float(), mask[b:b + 1].float())[0] for b in range(batch)])
        xd, md = x.to(DEV), mask.to(DEV)
        got = hip(xd, md)
        assert got.shape == x.shape and got.dtype == x.dtype
        print(assert_close(got, want, f"triattn c={c} h={h}", auto_scale=True), flush=True)
        assert torch.equal(got, hip(xd, md)), "run-to-run results differ"
        # mask=None and the fused residual
        got_n = hip(xd, None)
        want_n = torch.stack([ref(x[b:b + 1].float(), None)[0] for b in range(batch)])
        assert_close(got_n, want_n, "mask=None", auto_scale=True)
        xin = xd.clone()
        ops.triattn_forward(xin, md, hip._hip_attention_cache, h, starting, residual=xin, out=xin)
        assert_close(xin, x.float() + want, "residual in place", rel_fro=5e-3, auto_scale=True)


@pytest.mark.parametrize("flip", [False, True])
def test_template_batch_at_once_equals_templates_in_turn(flip):
    """A workspace of the batched size takes all templates through the kernels at once, one of the
    per-element size takes them in turn: same bits either way (c = 64, 4 templates)."""
    from kfold_amd import ops, primitives as P

    c, h, n, batch = 64, 4, 45, 4
    print(f"case template batch folded vs in turn flip={flip}", flush=True)
    g = torch.Generator().manual_seed(21)
    x = torch.randn(batch, n, n, c, generator=g).bfloat16().to(DEV)
    mask = (torch.rand(batch, n, n, generator=g) > 0.2).to(DEV)
    tm = getattr(P, "TriangleMultiplicationIncoming" if flip else "TriangleMultiplicationOutgoing")(c).eval()
    ta = getattr(P, "TriangleAttentionEndingNode" if flip else "TriangleAttentionStartingNode")(c, h).eval()
    for m, seed in ((tm, 5), (ta, 6)):
        synthetic.init_weights_(m, seed, std=0.08)
        _affine(m)
        m.to(DEV)
    with torch.no_grad():
        tm(x[:1], mask[:1]), ta(x[:1], mask[:1])       # packs the weights
        one, many = ops.workspace_bytes("trimul", N=n, C=c), ops.workspace_bytes("trimul", N=n, C=c, B=batch)
        assert many > one
        direction = "incoming" if flip else "outgoing"
        small = torch.empty(one + 256, dtype=torch.uint8, device=DEV)
        small = small[(-small.data_ptr()) % 256:][:one]
        a = ops.trimul_forward(x, mask, tm._hip_multiplication_cache, direction, workspace=small)
        b = ops.trimul_forward(x, mask, tm._hip_multiplication_cache, direction)
        assert torch.equal(a, b), "tri-mul: batch at once differs from elements in turn"
        one, many = ops.workspace_bytes("triattn", N=n, C=c, heads=h), ops.workspace_bytes("triattn", N=n, C=c, heads=h, B=batch)
        assert many > one
        small = torch.empty(one + 256, dtype=torch.uint8, device=DEV)
        small = small[(-small.data_ptr()) % 256:][:one]
        a = ops.triattn_forward(x, mask, ta._hip_attention_cache, h, not flip, workspace=small)
        b = ops.triattn_forward(x, mask, ta._hip_attention_cache, h, not flip)
        assert torch.equal(a, b), "tri-attn: batch at once differs from elements in turn"
        # the fused widths have no batched mode: same size either way
        assert ops.workspace_bytes("trimul", N=n, C=128, B=batch) == ops.workspace_bytes("trimul", N=n, C=128)


@pytest.mark.parametrize("direction", ["outgoing", "incoming"])
@pytest.mark.parametrize("n", [384, 768])
def test_trimul_c256_tiled_sizes(direction, n):
    """C = 256 at sizes whose padded planes take the 256 x 256 contraction tiles (N = 130 and
    below run on 128 x 128 tiles only) with 12 % padding; the oracle's einsum in full."""
    from kfold_amd import primitives as P
    from oracle import torch_path as O

    print(f"case trimul C=256 {direction} n={n}", flush=True)
    cls = "TriangleMultiplicationOutgoing" if direction == "outgoing" else "TriangleMultiplicationIncoming"
    ref = getattr(O, cls)(256).eval()
    synthetic.init_weights_(ref, 5)
    hip = getattr(P, cls)(256).eval()
    hip.load_state_dict(ref.state_dict())
    hip.to(DEV)
    z, _, pm = synthetic.pair_inputs(n, 256, synthetic.n_pad_for(n, 0.12), seed=n + 1)
    zb = z.bfloat16()
    with torch.no_grad():
        want = ref(zb.float(), pm)
        got = hip(zb.to(DEV), pm.to(DEV))
    print(assert_close(got, want, f"trimul C=256 {direction} n={n}"), flush=True)
    assert (got.cpu()[~pm] == 0).all()


@pytest.mark.parametrize("starting", [True, False])
def test_triattn_c64_templates_n384(starting):
    """The template stack's shape at a realistic length: c = 64, 4 heads x 16, 4 templates,
    N = 384 (12 key blocks; the bias of each template is its own).  Oracle on sampled rows of
    every template."""
    from kfold_amd import primitives as P
    from oracle import torch_path as O

    print(f"case triattn c=64 templates n=384 starting={starting}", flush=True)
    n, batch = 384, 4
    cls = "TriangleAttentionStartingNode" if starting else "TriangleAttentionEndingNode"
    ref = getattr(O, cls)(64, 4).eval()
    synthetic.init_weights_(ref, 17, std=0.08)
    hip = getattr(P, cls)(64, 4).eval()
    hip.load_state_dict(ref.state_dict())
    hip.to(DEV)
    g = torch.Generator().manual_seed(n)
    x = torch.randn(batch, n, n, 64, generator=g).bfloat16()
    masks = [synthetic.pair_mask_from_tokens(synthetic.token_mask(n, pad))[0] for pad in (0, 46, 7, 100)]
    mask = torch.stack(masks)
    rows = [0, 31, 32, 200, 283, 284, 337, 338, 383]
    with torch.no_grad():
        got = hip(x.to(DEV), mask.to(DEV)).float().cpu()
        for b in range(batch):
            xt = x[b:b + 1].float() if starting else x[b:b + 1].float().transpose(1, 2)
            mt = mask[b:b + 1].float() if starting else mask[b:b + 1].float().transpose(1, 2)
            xn = ref.layer_norm(xt)
            bias = ref.linear(xn).movedim(-1, -3).unsqueeze(-4)
            want = ref.mha(xn[:, rows], xn[:, rows], bias, mt[..., :, None, None, :][:, rows])[0]
            gb = (got[b] if starting else got[b].transpose(0, 1))[rows]
            print(assert_close(gb, want, f"triattn c=64 template {b}", auto_scale=True), flush=True)


@pytest.mark.parametrize("direction", ["outgoing", "incoming"])
@pytest.mark.parametrize("c,n,n_pad", [(64, 37, 5), (64, 70, 0), (96, 50, 6)])
def test_trimul_other_widths(direction, c, n, n_pad):
    """Triangle multiplication at the template stack's width (c = 64) and at another multiple of
    32: the path assembled from the token-track kernels and the contraction kernel."""
    from kfold_amd import ops, primitives as P
    from oracle import torch_path as O

    print(f"case trimul C={c} {direction} n={n}", flush=True)
    cls = "TriangleMultiplicationOutgoing" if direction == "outgoing" else "TriangleMultiplicationIncoming"
    ref = getattr(O, cls)(c).eval()
    synthetic.init_weights_(ref, 3, std=0.05)
    _affine(ref)
    hip = getattr(P, cls)(c).eval()
    hip.load_state_dict(ref.state_dict())
    hip.to(DEV)
    z, _, pm = synthetic.pair_inputs(n, c, n_pad, seed=n)
    if n == 70:         # a general (not outer-product) mask
        pm = torch.rand(1, n, n, generator=torch.Generator().manual_seed(5)) > 0.3
    zb = z.bfloat16()
    with torch.no_grad():
        want = ref(zb.float(), pm)
        zd, pmd = zb.to(DEV), pm.to(DEV)
        got = hip(zd, pmd)
        print(assert_close(got, want, f"trimul C={c} {direction}", auto_scale=True), flush=True)
        assert torch.equal(got, hip(zd, pmd)), "run-to-run results differ"
        zin = zd.clone()
        ops.trimul_forward(zin, pmd, hip._hip_multiplication_cache, direction, residual=zin, out=zin)
        assert_close(zin, zb.float() + want, "residual in place", rel_fro=5e-3, auto_scale=True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_template_stack_block_c64(dtype):
    """The whole Pairformer block of the apo template stack (model/modules/apo_module.py:107-172,
    :294-301: channel_z = 64, 4 triangle-attention heads of 16) over a batch of templates, in place,
    with the final mask."""
    from kfold_amd import modules as M
    from oracle import torch_path as O

    print(f"case template-stack block C=64 {dtype}", flush=True)
    ref = O.PairformerBlock(64, 4).eval()
    synthetic.init_weights_(ref, 21, std=0.05)
    hip = M.PairformerBlock(64, 4).eval()
    hip.load_state_dict(ref.state_dict())
    hip.to(DEV)
    n, batch = 44, 3
    g = torch.Generator().manual_seed(4)
    z = torch.randn(batch, n, n, 64, generator=g)
    pm = torch.stack([synthetic.pair_mask_from_tokens(synthetic.token_mask(n, pad))[0] for pad in (0, 5, 12)])
    zi = z.to(dtype)
    with torch.no_grad():
        zw = torch.stack([ref(zi[b:b + 1].float().clone(), pm[b:b + 1].float())[0] for b in range(batch)])
        zin = zi.to(DEV)
        zg = hip(zin, pm.to(DEV), inplace_output=True)
    assert zg.data_ptr() == zin.data_ptr()
    if dtype == torch.float32:
        print(assert_close(zg, zw, "template-stack block, fp32 stream", rel_fro=5e-3, auto_scale=True), flush=True)
    else:   # bf16 stream: five storage roundings of |z| up to ~5 on top of the kernel error
        print(assert_close(zg, zw, "template-stack block, bf16 stream", max_abs=8e-2, mean_abs=6e-3, rel_fro=8e-3),
              flush=True)
    assert (zg.cpu()[~pm] == 0).all()
