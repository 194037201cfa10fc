"""HIP Pairformer block / trunk vs the fp32 oracle."""

import pytest
import torch

from kfold_amd import synthetic
from tests.util import assert_close

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _blocks(num=1, seed=0, std=0.02):
    from kfold_amd import modules as M
    from oracle import torch_path as O

    ref = O.PairformerTrunk(num, row_chunk=32).eval()
    synthetic.init_weights_(ref, seed, std=std)
    hip = M.PairformerTrunk(num).eval()
    hip.load_state_dict(ref.state_dict())
    return ref, hip.to(DEV)


@pytest.mark.parametrize("n,frac", [(64, 0.0), (100, 0.15)])
def test_block_parity_and_masked_zero(n, frac):
    """Config 1 shape (N=64, all-ones mask) and a padded odd size, one block, bf16."""
    print(f"case block n={n} pad={frac}", flush=True)
    ref, hip = _blocks(1)
    z, tok, pm = synthetic.pair_inputs(n, 128, synthetic.n_pad_for(n, frac), seed=0)
    s = synthetic.single_inputs(n, 384, seed=1)
    zb, sb = z.bfloat16(), s.bfloat16()
    with torch.no_grad():
        zw, sw = ref(zb.float(), sb.float(), pm.float(), tok.float())
        zin, sin = zb.to(DEV), sb.to(DEV)
        zg, sg = hip(zin, sin, pm.to(DEV), tok.to(DEV))
    # The residual stream |z| ~ N(0,1) is stored in bf16 and rounded after each of the 5
    # in-place updates (as a bf16 z would be by the reference's own z.add_), so the absolute
    # error scales with |z|; the fp32-io test below holds the unscaled tolerances.
    assert_close(zg, zw, "block z", rel_fro=8e-3, auto_scale=True)
    assert_close(sg, sw, "block s", rel_fro=8e-3, auto_scale=True)
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
    from kfold_amd import modules as M

    print("case block f32", flush=True)
    ref, hip = _blocks(1, seed=2, std=0.05)
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


def test_trunk_three_blocks():
    print("case trunk x3", flush=True)
    ref, hip = _blocks(3, seed=5)
    n = 72
    z, tok, pm = synthetic.pair_inputs(n, 128, 9, seed=6)
    s = synthetic.single_inputs(n, 384, seed=7)
    zb, sb = z.bfloat16(), s.bfloat16()
    with torch.no_grad():
        zw, sw = ref(zb.float(), sb.float(), pm.float(), tok.float())
        zg, sg = hip(zb.to(DEV), sb.to(DEV), pm.to(DEV), tok.to(DEV))
    assert_close(zg, zw, "trunk z", rel_fro=1.5e-2, auto_scale=True)
    assert_close(sg, sw, "trunk s", rel_fro=1.5e-2, auto_scale=True)
    assert (zg.cpu()[~pm] == 0).all()
