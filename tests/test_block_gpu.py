"""HIP Pairformer block / trunk vs the oracle.

A bf16 residual stream is rounded after each in-place update, which alone moves ``z`` away
from the all-fp32 oracle by more than the north-star limits (|z| ~ N(0,1) reaches 4-6, where
bf16 steps are 2^-5).  The block tests therefore separate the two sources of error:

* stage by stage ("teacher forced"): every in-place update of the HIP block is compared, at
  the unscaled limits, with the fp32 oracle op applied to the very same bf16 input;
* end to end against the oracle run with a bf16-rounded stream, with the all-fp32 oracle as
  control (see ``tests.util.assert_stream_close``);
* with fp32 activations at the boundary (no storage rounding) the whole block meets the
  unscaled limits against the all-fp32 oracle.
"""

import pytest
import torch

from kfold_amd import synthetic
from tests.util import assert_close, assert_stream_close

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _blocks(num=1, seed=0, std=0.02, row_chunk=32):
    from kfold_amd import modules as M
    from oracle import torch_path as O

    ref = O.PairformerTrunk(num, row_chunk=row_chunk).eval()
    synthetic.init_weights_(ref, seed, std=std)
    stream = O.PairformerTrunk(num, row_chunk=row_chunk, stream_dtype=torch.bfloat16).eval()
    stream.load_state_dict(ref.state_dict())
    hip = M.PairformerTrunk(num).eval()
    hip.load_state_dict(ref.state_dict())
    return ref, stream, hip.to(DEV)


def pair_stages(ref_block, hip_block, pm, pm_dev):
    """(name, oracle update fn, HIP in-place fn) for the five updates of the pair track; the last
    one carries the block's final mask."""
    from kfold_amd import modules as M
    from kfold_amd.layers.transition import hip_transition

    rb, hb = ref_block.pair_block, hip_block.pair_block
    pmf = pm.float()
    return [
        ("tri_mul_out", lambda x: x + rb.tri_mul_out(x, pmf),
         lambda x: M._trimul_inplace(hb.tri_mul_out, x, pm_dev)),
        ("tri_mul_in", lambda x: x + rb.tri_mul_in(x, pmf),
         lambda x: M._trimul_inplace(hb.tri_mul_in, x, pm_dev)),
        ("tri_att_start", lambda x: x + rb.tri_att_start(x, pmf),
         lambda x: M._triattn_inplace(hb.tri_att_start, x, pm_dev)),
        ("tri_att_end", lambda x: x + rb.tri_att_end(x, pmf),
         lambda x: M._triattn_inplace(hb.tri_att_end, x, pm_dev)),
        ("transition_z + mask", lambda x: (x + rb.transition_z(x)) * pmf[..., None],
         lambda x: hip_transition(hb.transition_z, x, residual=x, mask=pm_dev, out=x)),
    ]


def check_stagewise(ref_block, hip_block, z_dev, pm, what):
    """Walk the pair track on the HIP stream ``z_dev`` (in place); before each update the oracle
    op is evaluated in fp32 on a copy of the stream's current values."""
    out = {}
    with torch.no_grad():
        for name, ref_fn, hip_fn in pair_stages(ref_block, hip_block, pm, pm.to(z_dev.device)):
            want = ref_fn(z_dev.float().cpu())
            hip_fn(z_dev)
            out[name] = assert_close(z_dev, want, f"{what} stage {name}", rel_fro=None)
    return out


@pytest.mark.parametrize("n,frac", [(64, 0.0), (100, 0.15)])
def test_block_parity_and_masked_zero(n, frac):
    """Config 1 shape (N=64, all-ones mask) and a padded odd size, one block, bf16."""
    print(f"case block n={n} pad={frac}", flush=True)
    ref, stream, hip = _blocks(1)
    z, tok, pm = synthetic.pair_inputs(n, 128, synthetic.n_pad_for(n, frac), seed=0)
    s = synthetic.single_inputs(n, 384, seed=1)
    zb, sb = z.bfloat16(), s.bfloat16()
    with torch.no_grad():
        zw, sw = ref(zb.float(), sb.float(), pm.float(), tok.float())
        zs, ss = stream(zb.float(), sb.float(), pm.float(), tok.float())
        zin, sin = zb.to(DEV), sb.to(DEV)
        zg, sg = hip(zin, sin, pm.to(DEV), tok.to(DEV))
    print(assert_stream_close(zg, zs, zw, "block z"), flush=True)
    print(assert_stream_close(sg, ss, sw, "block s"), flush=True)
    # every update on its own, unscaled limits
    check_stagewise(ref.blocks[0], hip.blocks[0], zb.to(DEV), pm, f"block n={n}")
    # masked positions are bit-exact zero
    assert (zg.cpu()[~pm] == 0).all()
    # in place like the reference's eval-mode adds
    assert zg.data_ptr() == zin.data_ptr() and sg.data_ptr() == sin.data_ptr()
    # valid outputs do not depend on what padded tokens hold
    if frac:
        nv = n - synthetic.n_pad_for(n, frac)
        z2 = zb.clone()
        z2[:, nv:] = 50.0
        z2[:, :, nv:] = -50.0
        with torch.no_grad():
            zg2, _ = hip(z2.to(DEV), sb.to(DEV), pm.to(DEV), tok.to(DEV))
        assert torch.equal(zg2[:, :nv, :nv], zg[:, :nv, :nv])


def test_block_f32_io_fresh_output_and_update_size():
    """fp32 activations at the boundary (config 1 dtype); the update itself, not only the
    residual stream, must match."""
    print("case block f32", flush=True)
    ref, _, hip = _blocks(1, seed=2, std=0.05)
    n = 48
    z, tok, pm = synthetic.pair_inputs(n, 128, 6, seed=3)
    s = synthetic.single_inputs(n, 384, seed=4)
    with torch.no_grad():
        zw, sw = ref(z.clone(), s.clone(), pm.float(), tok.float())
        blk = hip.blocks[0]
        zin = z.to(DEV)
        zg = blk.pair_block(zin, pm.to(DEV))             # fresh output tensor
        assert zg.data_ptr() != zin.data_ptr()
    valid = pm[0]
    upd_w = (zw - z)[0][valid]
    upd_g = (zg.cpu() - z)[0][valid]
    assert_close(upd_g, upd_w, "block update (fp32 io)", rel_fro=3e-2)
    assert_close(zg, zw, "block z (fp32 io)", rel_fro=3e-3)
    assert (zg.cpu()[~pm] == 0).all()


def test_config1_block_f32_io_all_ones_mask():
    """Config 1 exactly: N=64, fp32 z and s at the boundary, all-ones masks, std-0.02 weights."""
    print("case config 1", flush=True)
    ref, _, hip = _blocks(1)
    z, tok, pm = synthetic.pair_inputs(64, 128, 0, seed=0)
    s = synthetic.single_inputs(64, 384, seed=1)
    with torch.no_grad():
        zw, sw = ref(z.clone(), s.clone(), pm.float(), tok.float())
        zg, sg = hip(z.to(DEV), s.to(DEV), pm.to(DEV), tok.to(DEV))
    print(assert_close(zg, zw, "config 1 z", rel_fro=3e-3), flush=True)
    print(assert_close(sg, sw, "config 1 s", rel_fro=3e-3), flush=True)


def test_trunk_three_blocks():
    print("case trunk x3", flush=True)
    ref, stream, hip = _blocks(3, seed=5)
    n = 72
    z, tok, pm = synthetic.pair_inputs(n, 128, 9, seed=6)
    s = synthetic.single_inputs(n, 384, seed=7)
    zb, sb = z.bfloat16(), s.bfloat16()
    with torch.no_grad():
        zw, sw = ref(zb.float(), sb.float(), pm.float(), tok.float())
        zs, ss = stream(zb.float(), sb.float(), pm.float(), tok.float())
        zg, sg = hip(zb.to(DEV), sb.to(DEV), pm.to(DEV), tok.to(DEV))
    print(assert_stream_close(zg, zs, zw, "trunk z", max_flip_frac=2e-3, n_adds=15), flush=True)
    print(assert_stream_close(sg, ss, sw, "trunk s", max_flip_frac=2e-3, n_adds=6), flush=True)
    assert (zg.cpu()[~pm] == 0).all()
    # the two-stream schedule (single track of block b beside the pair track of block b+1) gives
    # the same bits as the serial one
    from kfold_amd import modules as M
    with torch.no_grad():
        zs_, ss_ = M.run_blocks(list(hip.blocks), zb.to(DEV), sb.to(DEV), pm.to(DEV), tok.to(DEV), side=None)
        torch.cuda.synchronize()
    assert hip.overlap_tracks and torch.equal(zs_, zg) and torch.equal(ss_, sg)
    # the same three blocks with an fp32 stream: no storage rounding, unscaled limits end to end
    with torch.no_grad():
        zf, sf = hip(zb.float().to(DEV), sb.float().to(DEV), pm.to(DEV), tok.to(DEV))
    print(assert_close(zf, zw, "trunk z (fp32 stream)", rel_fro=8e-3), flush=True)
    print(assert_close(sf, sw, "trunk s (fp32 stream)", rel_fro=8e-3), flush=True)


def test_triangular_block():
    """The shipping trunk block (tri-mul out, tri-mul in, transition x4, no final mask) at
    c_z = 128: bf16 stream stage by stage, fp32 stream end to end."""
    from kfold_amd import modules as M
    from kfold_amd.layers.transition import hip_transition
    from oracle import torch_path as O

    print("case triangular block", flush=True)
    ref = O.TriangularBlock(128).eval()
    synthetic.init_weights_(ref, 11)
    hip = M.TriangularBlock(128).eval()
    hip.load_state_dict(ref.state_dict())
    hip.to(DEV)
    n = 90
    z, _, pm = synthetic.pair_inputs(n, 128, 11, seed=12)
    zb = z.bfloat16()
    with torch.no_grad():
        zw = ref(zb.float(), pm.float())
        zin = zb.float().to(DEV)
        zg = hip(zin, pm.to(DEV))
        assert zg.data_ptr() == zin.data_ptr()           # in place, like the reference in eval mode
        print(assert_close(zg, zw, "triangular block (fp32 stream)", rel_fro=5e-3), flush=True)
        # padded positions are NOT zeroed by this block (no final mask): they hold z + transition(z)
        assert (zg.cpu()[~pm].abs().sum() > 0)
        # bf16 stream, each update against the oracle op on the same input
        zd = zb.to(DEV)
        pmd, pmf = pm.to(DEV), pm.float()
        stages = [
            (lambda x: x + ref.tri_mul_out(x, pmf), lambda x: M._trimul_inplace(hip.tri_mul_out, x, pmd)),
            (lambda x: x + ref.tri_mul_in(x, pmf), lambda x: M._trimul_inplace(hip.tri_mul_in, x, pmd)),
            (lambda x: x + ref.transition_z(x), lambda x: hip_transition(hip.transition_z, x, residual=x, out=x)),
        ]
        for i, (rf, hf) in enumerate(stages):
            want = rf(zd.float().cpu())
            hf(zd)
            assert_close(zd, want, f"triangular block stage {i}", rel_fro=None)
        # the module call gives the same bits as the stage walk
        assert torch.equal(hip(zb.to(DEV), pmd), zd)


def test_empty_inputs_give_empty_outputs():
    """No tokens, no batch elements, no samples, no windows: every module returns an empty tensor
    of the input's shape, as the reference's torch path does, without a kernel launch."""
    from kfold_amd import layers, modules as M, primitives as P

    print("case empty inputs", flush=True)
    mk = lambda m: synthetic.init_weights_(m.eval(), 0).to(DEV)
    z0 = torch.zeros(1, 0, 0, 128).bfloat16().to(DEV)
    m0 = torch.zeros(1, 0, 0, dtype=torch.bool).to(DEV)
    zb = torch.zeros(0, 8, 8, 128).bfloat16().to(DEV)
    mb = torch.zeros(0, 8, 8, dtype=torch.bool).to(DEV)
    f = lambda *shape: torch.zeros(*shape).to(DEV)
    with torch.no_grad():
        for mod in (mk(P.TriangleMultiplicationOutgoing(128)), mk(P.TriangleMultiplicationIncoming(128)),
                    mk(P.TriangleAttentionStartingNode(128, 4)), mk(P.TriangleAttentionEndingNode(128, 4)),
                    mk(P.TriangleMultiplicationOutgoing(64)), mk(P.TriangleAttentionStartingNode(64, 4))):
            c = mod.linear_p_in.weight.shape[1] if hasattr(mod, "linear_p_in") else mod.c_in
            assert mod(z0[..., :c], m0).shape == (1, 0, 0, c)
            assert mod(zb[..., :c], mb).shape == (0, 8, 8, c)
        assert mk(layers.Transition(128, 2))(f(0, 128)).shape == (0, 128)
        assert mk(layers.Transition(384, 4))(f(0, 384)).shape == (0, 384)
        apb = mk(layers.SelfAttentionPairBias(768, 16, 384, "diffusion_global"))
        assert apb(f(1, 2, 0, 768), f(1, 2, 0, 384), f(1, 1, 16, 0, 0), m0.reshape(1, 1, 0)).shape == (1, 2, 0, 768)
        assert apb(f(1, 0, 8, 768), f(1, 0, 8, 384), f(1, 1, 16, 8, 8),
                   torch.ones(1, 1, 8, dtype=torch.bool).to(DEV)).shape == (1, 0, 8, 768)
        cross = mk(layers.CrossAttentionPairBias(128, 4, 128))
        assert cross(f(2, 0, 32, 128), f(2, 0, 128, 128), f(2, 0, 32, 128), f(2, 0, 128, 128), f(1, 0, 4, 32, 128),
                     torch.ones(1, 0, 128, dtype=torch.bool).to(DEV)).shape == (2, 0, 32, 128)
        assert M.ParcaeStep(128).eval().to(DEV)(f(1, 0, 0, 128), f(1, 0, 0, 128)).shape == (1, 0, 0, 128)
        zz, ss = mk(M.PairSingleBlock())(z0, torch.zeros(1, 0, 384).bfloat16().to(DEV), m0,
                                        torch.zeros(1, 0, dtype=torch.bool).to(DEV))
        assert zz.shape == (1, 0, 0, 128) and ss.shape == (1, 0, 384)


@pytest.mark.parametrize("c,heads,batch,n", [(128, 4, 1, 70), (128, 4, 2, 37), (64, 4, 3, 45)])
def test_pair_block_in_one_c_call(c, heads, batch, n):
    """kfh_pair_block_forward (the pair track of a block in one C call, for callers without the Python
    layer) against the module: same kernels, same bits; fp32 and bf16 tensors."""
    from kfold_amd import _lib, modules as M

    print(f"case pair block in one C call c={c} batch={batch} n={n}", flush=True)
    blk = synthetic.init_weights_(M.PairformerBlock(c, heads).eval(), 4, std=0.05).to(DEV)
    g = torch.Generator().manual_seed(n)
    pm = torch.stack([synthetic.pair_mask_from_tokens(synthetic.token_mask(n, 3 * b))[0] for b in range(batch)]).to(DEV)
    L = _lib.lib()
    for dtype in (torch.bfloat16, torch.float32):
        z = torch.randn(batch, n, n, c, generator=g).to(dtype).to(DEV)
        with torch.no_grad():
            want = blk(z.clone(), pm, inplace_output=True)
        blobs = [blk.tri_mul_out._hip_multiplication_cache, blk.tri_mul_in._hip_multiplication_cache,
                 blk.tri_att_start._hip_attention_cache, blk.tri_att_end._hip_attention_cache,
                 blk.transition_z._hip_transition_cache]
        need = L.kfh_pair_block_workspace_bytes(batch, n, c, heads, 2)
        assert need > 0
        ws = torch.empty(need + 256, dtype=torch.uint8, device=DEV)
        ws = ws[(-ws.data_ptr()) % 256:][:need]
        got = z.clone()
        m8 = pm.contiguous().view(torch.uint8)
        io = _lib.KFH_BF16 if dtype == torch.bfloat16 else _lib.KFH_F32
        stream = torch.cuda.current_stream().cuda_stream
        _lib.check(L.kfh_pair_block_forward(got.data_ptr(), m8.data_ptr(), *[b.data_ptr() for b in blobs], ws.data_ptr(),
                                            need, batch, n, c, heads, 2, 1e-5, io, stream))
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"{dtype}"
        assert (got.float().cpu()[~pm.cpu()] == 0).all()
    assert L.kfh_pair_block_workspace_bytes(1, n, 48, 4, 2) == 0


@pytest.mark.parametrize("batch,n", [(1, 70), (2, 37)])
def test_single_track_in_one_c_call(batch, n):
    """kfh_single_track_forward (pair bias from z, attention, transition, in place on s) against the
    module's single track: same kernels, same bits."""
    from kfold_amd import _lib, modules as M

    print(f"case single track in one C call batch={batch} n={n}", flush=True)
    blk = synthetic.init_weights_(M.PairSingleBlock().eval(), 7, std=0.05).to(DEV)
    g = torch.Generator().manual_seed(n)
    tok = torch.stack([synthetic.token_mask(n, 4 * b)[0] for b in range(batch)]).to(DEV)
    L = _lib.lib()
    for dtype in (torch.bfloat16, torch.float32):
        z = torch.randn(batch, n, n, 128, generator=g).to(dtype).to(DEV)
        s = torch.randn(batch, n, 384, generator=g).to(dtype).to(DEV)
        want = s.clone()
        with torch.no_grad():
            blk.single_track(z, want, tok)
        blobs = [blk._hip_pair_bias_cache, blk.attention._hip_apb_cache, blk.transition._hip_transition_cache]
        need = L.kfh_single_track_workspace_bytes(batch, n, 128, 384, 16, 4)
        assert need > 0
        ws = torch.empty(need + 256, dtype=torch.uint8, device=DEV)
        ws = ws[(-ws.data_ptr()) % 256:][:need]
        got = s.clone()
        io = _lib.KFH_BF16 if dtype == torch.bfloat16 else _lib.KFH_F32
        _lib.check(L.kfh_single_track_forward(z.data_ptr(), got.data_ptr(), tok.contiguous().view(torch.uint8).data_ptr(),
                                              *[b.data_ptr() for b in blobs], ws.data_ptr(), need, batch, n, 128, 384, 16,
                                              4, 1e-5, io, torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"{dtype}"
    assert L.kfh_single_track_workspace_bytes(1, n, 64, 384, 16, 4) == 0
