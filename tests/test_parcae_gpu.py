"""HIP Parcae recurrence step vs the fp32 oracle."""

import pytest
import torch

from kfold_amd import synthetic
from tests.util import assert_close

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _pair(C, seed):
    from kfold_amd import modules as M
    from oracle import torch_path as O

    ref = O.ParcaeStep(C).eval()
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        ref.parcae_log_a.copy_(0.3 * torch.randn(C, generator=g))
        ref.parcae_log_delta.add_(0.5 * torch.randn(C, generator=g))
        ref.parcae_b_cont.add_(0.05 * torch.randn(C, C, generator=g))
        ref.layernorm_z.weight.copy_(1 + 0.2 * torch.randn(C, generator=g))
        ref.layernorm_z.bias.copy_(0.1 * torch.randn(C, generator=g))
    hip = M.ParcaeStep(C).eval()
    hip.load_state_dict(ref.state_dict())
    return ref, hip.to(DEV)


@pytest.mark.parametrize("C", [128, 256])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_parcae_step_parity(C, dtype):
    print(f"case parcae C={C} {dtype}", flush=True)
    ref, hip = _pair(C, 3)
    n = 45                                           # 2025 rows: not a multiple of the 128-row tile
    g = torch.Generator().manual_seed(4)
    z = torch.randn(1, n, n, C, generator=g).to(dtype)
    u = (2.0 * torch.randn(1, n, n, C, generator=g) + 0.5).to(dtype)
    with torch.no_grad():
        want = ref(z.float(), u.float())
        zd = z.to(DEV)
        got = hip(zd, u.to(DEV), inplace=False)
        assert got.data_ptr() != zd.data_ptr() and torch.equal(zd.cpu(), z)
        if dtype == torch.float32:
            print(assert_close(got, want, f"parcae C={C} f32", rel_fro=5e-3), flush=True)
        else:
            # the state itself is stored in bf16: one storage rounding of an O(1) value
            print(assert_close(got, want, f"parcae C={C} bf16", rel_fro=5e-3), flush=True)
        got2 = hip(zd, u.to(DEV))                    # in place on z
        assert got2.data_ptr() == zd.data_ptr() and torch.equal(got2, got)
    # the update term alone (a * z removed) within the unscaled limits
    a, _ = ref.dynamics()
    upd_w = want - a * z.float()
    upd_g = got.float().cpu() - a * z.float()
    if dtype == torch.float32:
        assert_close(upd_g, upd_w.detach(), "parcae injected term", rel_fro=1e-2)


def test_parcae_module_names_and_errors():
    from kfold_amd import _lib, modules as M
    from oracle import torch_path as O

    assert sorted(M.ParcaeStep(128).state_dict()) == sorted(O.ParcaeStep(128).state_dict())
    assert set(M.ParcaeStep(128).state_dict()) == {"layernorm_z.weight", "layernorm_z.bias", "parcae_log_a",
                                                     "parcae_log_delta", "parcae_b_cont"}
    L = _lib.lib()
    assert L.kfh_parcae_packed_bytes(128) > 0 and L.kfh_parcae_packed_bytes(64) == 0
    hip = M.ParcaeStep(128).eval().to(DEV)
    z = torch.zeros(4, 128, device=DEV)
    with torch.no_grad(), pytest.raises(ValueError):
        hip(z, torch.zeros(4, 64, device=DEV))


def test_parcae_trunk_recurrence_and_reference_named_weights():
    """Two recycles of the trunk recurrence at c_z = 256 (2 + 3 triangular blocks), weights loaded
    from a state dict that carries the reference model's key names."""
    from kfold_amd import modules as M
    from kfold_amd.runtime import load_reference_weights
    from oracle import torch_path as O

    print("case parcae trunk", flush=True)
    C, n = 256, 40
    ref = O.ParcaeTrunk(C, lm_blocks=2, main_blocks=3).eval()
    synthetic.init_weights_(ref, 21)
    with torch.no_grad():
        ref.parcae_b_cont.copy_(torch.eye(C) + 0.05 * torch.randn(C, C, generator=torch.Generator().manual_seed(2)))
        ref.parcae_log_a.zero_()
        ref.parcae_log_delta.fill_(0.2)
    # a checkpoint of the whole model: the trunk's entries sit beside ones with no hip counterpart
    ckpt = {k: v.clone() for k, v in ref.state_dict().items()}
    ckpt["input_embedder.linear.weight"] = torch.zeros(3, 3)
    ckpt["refine_stack.blocks.0.tri_mul_out.linear_p_in.weight"] = torch.zeros(2 * C, C)
    hip = M.ParcaeTrunk(C, lm_blocks=2, main_blocks=3).eval()
    used = load_reference_weights(hip, ckpt)
    assert "main_stack.blocks.2.transition_z.linear_out.weight" in used and len(used) == len(hip.state_dict())
    with pytest.raises(KeyError):
        load_reference_weights(M.TrianglularStack(C, 1), ckpt, prefix="no_such_stack.")
    sub = M.TrianglularStack(C, 3).eval()
    load_reference_weights(sub, ckpt, prefix="main_stack.")
    assert torch.equal(sub.blocks[1].tri_mul_in.linear_g_in.weight, ref.main_stack.blocks[1].tri_mul_in.linear_g_in.weight)
    hip.to(DEV)
    g = torch.Generator().manual_seed(5)
    z0 = (0.3 * torch.randn(1, n, n, C, generator=g))
    zin = torch.randn(1, n, n, C, generator=g)
    zlm = torch.randn(1, n, n, C, generator=g)
    pm = synthetic.pair_mask_from_tokens(synthetic.token_mask(n, 5))
    with torch.no_grad():
        want = ref(z0.clone(), zin, zlm, pm.float(), num_recycles=1)
        got = hip(z0.to(DEV), zin.to(DEV), zlm.to(DEV), pm.to(DEV), num_recycles=1)
    # a wiring test, not a benchmark configuration: 12 chained stages on an O(1) state, so the
    # absolute limits scale with the state's RMS; the relative gate is the sharp one
    print(assert_close(got, want, "parcae trunk, fp32 stream, 2 recycles", rel_fro=8e-3, auto_scale=True), flush=True)
