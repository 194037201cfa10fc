"""HIP triangle multiplication vs the fp32 oracle (through the C ABI, on the GPU)."""

import pytest
import torch

from kfold_amd import synthetic
from tests.util import assert_close

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _modules(direction, seed=0, ln_affine=False):
    from kfold_amd import primitives as P
    from oracle import torch_path as O

    cls = "TriangleMultiplicationOutgoing" if direction == "outgoing" else "TriangleMultiplicationIncoming"
    ref = getattr(O, cls)(128).eval()
    synthetic.init_weights_(ref, seed)
    if ln_affine:   # exercise gamma/beta handling, which the benchmark init (1/0) does not
        g = torch.Generator().manual_seed(seed + 100)
        with torch.no_grad():
            for ln in (ref.layernorm_in, ref.layernorm_out):
                ln.weight.copy_(1 + 0.2 * torch.randn(128, generator=g))
                ln.bias.copy_(0.1 * torch.randn(128, generator=g))
    hip = getattr(P, cls)(128).eval()
    hip.load_state_dict(ref.state_dict())
    return ref, hip.to(DEV)


def _run(ref, hip, z, mask, dtype):
    with torch.no_grad():
        want = ref(z.to(dtype).float(), mask)      # oracle sees the same rounded input
        got = hip(z.to(dtype).to(DEV), mask.to(DEV))
    assert got.dtype == dtype and got.shape == z.shape
    return got, want


@pytest.mark.parametrize("direction", ["outgoing", "incoming"])
@pytest.mark.parametrize("n,n_pad", [(64, 0), (37, 5), (130, 17), (1, 0), (256, 30)])
def test_trimul_parity_bf16(direction, n, n_pad):
    print(f"case trimul {direction} n={n} pad={n_pad}", flush=True)
    ref, hip = _modules(direction, ln_affine=(n == 37))
    z, _, pm = synthetic.pair_inputs(n, 128, n_pad, seed=n)
    got, want = _run(ref, hip, z, pm, torch.bfloat16)
    assert_close(got, want, f"trimul {direction} n={n}")


@pytest.mark.parametrize("direction", ["outgoing", "incoming"])
def test_trimul_general_mask_and_f32_io(direction):
    """Arbitrary (non outer-product) mask, fp32 activations at the boundary."""
    print(f"case trimul general mask {direction}", flush=True)
    ref, hip = _modules(direction, seed=3)
    n = 96
    z, _, _ = synthetic.pair_inputs(n, 128, 0, seed=11)
    mask = torch.rand(1, n, n, generator=torch.Generator().manual_seed(5)) > 0.3
    got, want = _run(ref, hip, z, mask, torch.float32)
    assert_close(got, want, f"trimul {direction} f32 io")


@pytest.mark.parametrize("direction", ["outgoing", "incoming"])
def test_trimul_config2_n384(direction):
    """Benchmark config 2: N=384, last 38 tokens padded, bf16."""
    print(f"case trimul config2 {direction}", flush=True)
    ref, hip = _modules(direction)
    z, _, pm = synthetic.pair_inputs(384, 128, 38, seed=0)
    got, want = _run(ref, hip, z, pm, torch.bfloat16)
    print(assert_close(got, want, f"trimul config2 {direction}"), flush=True)
    # masked (padded) positions: the op itself gives p_out(beta_out) * gate = 0 because beta = 0
    assert (got.cpu()[~pm.expand_as(pm)] == 0).all()


def test_trimul_batch_residual_determinism():
    from kfold_amd import ops

    print("case trimul batch/residual/determinism", flush=True)
    ref, hip = _modules("outgoing", seed=7)
    n = 48
    gen = torch.Generator().manual_seed(2)
    z = torch.randn(2, n, n, 128, generator=gen).to(torch.bfloat16)
    mask = torch.rand(2, n, n, generator=gen) > 0.2
    with torch.no_grad():
        want = torch.stack([ref(z[b:b + 1].float(), mask[b:b + 1])[0] for b in range(2)])
        zd, md = z.to(DEV), mask.to(DEV)
        got = hip(zd, md)
        assert_close(got, want, "trimul batch")
        again = hip(zd, md)
        assert torch.equal(got, again), "run-to-run results differ"
        # fused residual, in place: z += update
        blob = hip._hip_multiplication_cache
        zin = zd.clone()
        ops.trimul_forward(zin, md, blob, "outgoing", residual=zin, out=zin)
        assert_close(zin, z.float() + want, "trimul residual in place", rel_fro=5e-3)


def test_trimul_weight_cache_invalidation_and_errors():
    print("case trimul cache", flush=True)
    ref, hip = _modules("incoming", seed=9)
    z, _, pm = synthetic.pair_inputs(32, 128, 0, seed=4)
    zd, md = z.to(torch.bfloat16).to(DEV), pm.to(DEV)
    with torch.no_grad():
        a = hip(zd, md)
        key0 = hip._hip_multiplication_cache_key
        hip.linear_p_out.weight.mul_(2.0)            # in-place update bumps _version
        b = hip(zd, md)
        assert hip._hip_multiplication_cache_key != key0
        assert_close(b, 2 * a.float(), "cache invalidation", rel_fro=1e-2)
    with pytest.raises(RuntimeError):                # inference-only, like the triton backend
        with torch.enable_grad():
            hip(zd, md)


def test_cpu_tensors_are_rejected():
    _, hip = _modules("incoming", seed=9)
    z, _, pm = synthetic.pair_inputs(32, 128, 0, seed=4)
    with torch.no_grad(), pytest.raises(RuntimeError):
        hip(z.to(torch.bfloat16), pm)                # CPU tensor


def test_caller_workspace_shared_by_consecutive_ops():
    """One scratch buffer passed to triangle multiplication and triangle attention in turn (its
    contents are whatever the previous op left) gives the results of per-call allocations."""
    from kfold_amd import ops
    from kfold_amd import primitives as P

    print("case caller workspace shared by tri-mul and tri-attn", flush=True)
    n = 72
    tm = P.TriangleMultiplicationIncoming(128).eval()
    ta = P.TriangleAttentionStartingNode(128, 4).eval()
    synthetic.init_weights_(tm, 1)
    synthetic.init_weights_(ta, 2)
    tm, ta = tm.to(DEV), ta.to(DEV)
    z, _, pm = synthetic.pair_inputs(n, 128, 9, seed=4)
    zd, md = z.to(torch.bfloat16).to(DEV), pm.to(DEV)
    with torch.no_grad():
        want_tm, want_ta = tm(zd, md), ta(zd, md)            # packs the weights, allocates per call
        need = max(ops.workspace_bytes("trimul", N=n, C=128), ops.workspace_bytes("triattn", N=n, C=128, heads=4))
        raw = torch.full((need + 256,), 0xA5, dtype=torch.uint8, device=DEV)
        ws = raw[(-raw.data_ptr()) % 256:][:need]        # the library asks for 256-byte alignment
        for _ in range(2):
            got_tm = ops.trimul_forward(zd, md, tm._hip_multiplication_cache, "incoming", workspace=ws)
            got_ta = ops.triattn_forward(zd, md, ta._hip_attention_cache, 4, True, workspace=ws)
            assert torch.equal(got_tm, want_tm) and torch.equal(got_ta, want_ta)
        with pytest.raises(ValueError, match="needs"):
            ops.trimul_forward(zd, md, tm._hip_multiplication_cache, "incoming", workspace=ws[:1024])
