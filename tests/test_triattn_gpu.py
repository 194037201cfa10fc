"""HIP triangle attention vs the fp32 oracle (through the C ABI, on the GPU)."""

import pytest
import torch

from kfold_amd import synthetic
from tests.util import assert_close, errors

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _modules(starting, seed=0, ln_affine=False, std=0.02):
    from kfold_amd import primitives as P
    from oracle import torch_path as O

    cls = "TriangleAttentionStartingNode" if starting else "TriangleAttentionEndingNode"
    ref = getattr(O, cls)(128, 4, row_chunk=64).eval()
    synthetic.init_weights_(ref, seed, std=std)
    if ln_affine:
        g = torch.Generator().manual_seed(seed + 100)
        with torch.no_grad():
            ref.layer_norm.weight.copy_(1 + 0.2 * torch.randn(128, generator=g))
            ref.layer_norm.bias.copy_(0.1 * torch.randn(128, generator=g))
    hip = getattr(P, cls)(128, 4).eval()
    hip.load_state_dict(ref.state_dict())
    return ref, hip.to(DEV)


def _run(ref, hip, x, mask, dtype):
    with torch.no_grad():
        want = ref(x.to(dtype).float(), None if mask is None else mask.float())
        got = hip(x.to(dtype).to(DEV), None if mask is None else mask.to(DEV))
    assert got.dtype == dtype and got.shape == x.shape
    return got, want


@pytest.mark.parametrize("starting", [True, False])
@pytest.mark.parametrize("n,n_pad", [(64, 0), (37, 5), (130, 17), (1, 0), (256, 30)])
def test_triattn_parity_bf16(starting, n, n_pad):
    print(f"case triattn starting={starting} n={n} pad={n_pad}", flush=True)
    # larger weights at n=37 make the softmax far from uniform and the bias matter
    ref, hip = _modules(starting, ln_affine=(n == 37), std=0.1 if n == 37 else 0.02)
    x, _, pm = synthetic.pair_inputs(n, 128, n_pad, seed=n)
    got, want = _run(ref, hip, x, pm, torch.bfloat16)
    # rows whose keys are all masked (padded tokens) follow the same uniform-attention rule
    assert_close(got, want, f"triattn starting={starting} n={n}",
                 rel_fro=4e-2 if n == 37 else 2e-2)


@pytest.mark.parametrize("starting", [True, False])
def test_triattn_general_mask_none_mask_f32_io(starting):
    print(f"case triattn general mask starting={starting}", flush=True)
    ref, hip = _modules(starting, seed=3, std=0.05)
    n = 96
    x, _, _ = synthetic.pair_inputs(n, 128, 0, seed=11)
    mask = torch.rand(1, n, n, generator=torch.Generator().manual_seed(5)) > 0.3
    mask[0, 7, :] = False     # fully masked row (starting) ...
    mask[0, :, 9] = False     # ... and column (a fully masked "row" of the ending node)
    got, want = _run(ref, hip, x, mask, torch.float32)
    assert_close(got, want, f"triattn starting={starting} f32 io, general mask")
    got, want = _run(ref, hip, x, None, torch.float32)
    assert_close(got, want, f"triattn starting={starting} mask=None")


@pytest.mark.parametrize("starting", [True, False])
def test_triattn_config3_n512(starting):
    """Benchmark config 3: N=512, key mask zeroing the last 64 tokens, bf16."""
    print(f"case triattn config3 starting={starting}", flush=True)
    ref, hip = _modules(starting)
    x, _, pm = synthetic.pair_inputs(512, 128, 64, seed=0)
    got, want = _run(ref, hip, x, pm, torch.bfloat16)
    print(assert_close(got, want, f"triattn config3 starting={starting}"), flush=True)


def test_triattn_ending_is_transposed_starting_batch_residual_determinism():
    from kfold_amd import ops

    print("case triattn invariants", flush=True)
    ref, hs = _modules(True, seed=7, std=0.05)
    _, he = _modules(False, seed=7, std=0.05)
    n = 80
    gen = torch.Generator().manual_seed(2)
    x = torch.randn(2, n, n, 128, generator=gen).to(torch.bfloat16)
    mask = torch.rand(2, n, n, generator=gen) > 0.2
    xd, md = x.to(DEV), mask.to(DEV)
    with torch.no_grad():
        want = torch.stack([ref(x[b:b + 1].float(), mask[b:b + 1].float())[0] for b in range(2)])
        got = hs(xd, md)
        assert_close(got, want, "triattn batch")
        assert torch.equal(got, hs(xd, md)), "run-to-run results differ"
        # ending(x, m) == starting(x^T, m^T)^T, bit for bit: same arithmetic, different strides
        e = he(xd, md)
        s_t = hs(xd.transpose(1, 2).contiguous(), md.transpose(1, 2).contiguous()).transpose(1, 2)
        assert torch.equal(e, s_t)
        blob = hs._hip_attention_cache
        xin = xd.clone()
        ops.triattn_forward(xin, md, blob, 4, True, residual=xin, out=xin)
        assert_close(xin, x.float() + want, "triattn residual in place", rel_fro=5e-3)


def test_triattn_long_sequence_sampled_rows():
    """N = 1248 (39 key blocks: beyond the LDS strip of the short-sequence attention kernel, so
    the staged kernel runs).  The oracle is evaluated on a sample of rows only: rows are
    independent given the pair bias, which is computed for the whole tensor."""
    print("case triattn n=1248 sampled rows", flush=True)
    n, n_pad = 1248, 40
    ref, hip = _modules(True, seed=5)
    x, _, pm = synthetic.pair_inputs(n, 128, n_pad, seed=21)
    xb = x.to(torch.bfloat16)
    rows = [0, 1, 617, 1207, 1208, 1247]          # valid rows, the last valid row, padded rows
    with torch.no_grad():
        got = hip(xb.to(DEV), pm.to(DEV))[0, rows].float().cpu()
        xn = ref.layer_norm(xb.float())
        bias = ref.linear(xn).movedim(-1, -3).unsqueeze(-4)
        mask5 = pm.float()[..., :, None, None, :]
        want = ref.mha(xn[:, rows], xn[:, rows], bias, mask5[:, rows])[0]
    assert_close(got, want, "triattn n=1248 sampled rows")


@pytest.mark.parametrize("shift", [-256.0, 256.0, 60.0])
def test_triattn_logits_far_from_zero(shift):
    """A pair bias that is a large constant for every (query, key): the softmax is invariant to it,
    but exp2 of the raw logits under- or overflows, so the kernel has to fall back to the exact
    running-maximum path (negative shift) or move the maximum on the first block (positive)."""
    print(f"case triattn bias shift {shift}", flush=True)
    ref, hip = _modules(True, seed=9, std=0.05)
    with torch.no_grad():
        # LN(x) sums to 128 over the channels (gamma = 1, beta = 1), so a constant weight gives
        # bias = shift for every head, query and key: exactly representable in the bf16 bias
        # tiles, while q.k still varies
        ref.layer_norm.bias.fill_(1.0)
        ref.linear.weight.fill_(shift / 128.0)
    hip.load_state_dict(ref.state_dict())
    n = 96
    x, _, pm = synthetic.pair_inputs(n, 128, 9, seed=13)
    got, want = _run(ref, hip, x, pm, torch.bfloat16)
    assert_close(got, want, f"triattn bias shift {shift}", auto_scale=True)


def test_triattn_fully_masked_rows_with_large_varying_logits():
    """Large logits (|q.k| beyond 100) and rows whose keys are all masked.

    Rows with a valid key: at logits this size the rounding of the MFMA operands to bf16 (2^-9
    relative on q and k, i.e. a few tenths in an exponent of 100) moves the result away from an
    all-fp32 evaluation by far more than the benchmark tolerance.  That this is operand rounding
    and nothing else is shown by the oracle's rounded-operand mode (same formulas, every matrix
    operand rounded to bf16, fp32 sums): it is as far from the fp32 oracle as the kernel is, and
    the kernel matches IT at the unscaled limits.

    Rows whose keys are all masked (padded query rows; the block's final mask zeroes them):
    the reference adds a finite -1e9 to every masked logit in fp32 (triangle_attention.py:328):
    the spacing of fp32 at 1e9 is 64, so logits below 32 in magnitude vanish in that sum and the
    row attends uniformly, while larger ones leave a residue that is a multiple of 64 (weights
    then differ by factors of e^64 and flip with the last bit of q.k).  The kernel attends
    uniformly over the N keys in every fully masked row, whatever the logits: identical to the
    reference while |q.k|, |bias| < 32, a stated deviation beyond."""
    print("case triattn fully masked rows, large varying logits", flush=True)
    ref, hip = _modules(True, seed=21, std=0.02)
    g = torch.Generator().manual_seed(22)
    with torch.no_grad():
        for w in (ref.mha.linear_q.weight, ref.mha.linear_k.weight):
            w.copy_(0.5 * torch.randn(w.shape, generator=g))        # |q.k| reaches ~150
        ref.linear.weight.copy_(0.5 * torch.randn(ref.linear.weight.shape, generator=g))
        for w in (ref.mha.linear_v.weight, ref.mha.linear_o.weight, ref.mha.linear_g.weight):
            w.copy_(0.1 * torch.randn(w.shape, generator=g))
    hip.load_state_dict(ref.state_dict())
    n = 70
    x, _, _ = synthetic.pair_inputs(n, 128, 0, seed=23)
    mask = torch.rand(1, n, n, generator=g) > 0.3
    dead = [5, 33, 69]
    mask[0, dead, :] = False
    xb = x.to(torch.bfloat16)
    with torch.no_grad():
        got = hip(xb.to(DEV), mask.to(DEV)).float().cpu()
        want = ref(xb.float(), mask.float())
        ref.mha.operand_dtype = torch.bfloat16
        want_rounded = ref(xb.float(), mask.float())
        ref.mha.operand_dtype = None
        xn = ref.layer_norm(xb.float())
        q = ref.mha.linear_q(xn[0, dead]).unflatten(-1, (4, 32)) / 32 ** 0.5
        k = ref.mha.linear_k(xn[0, dead]).unflatten(-1, (4, 32))
        assert torch.einsum("rqhd,rkhd->rhqk", q, k).abs().max() > 32     # residues do occur
        live = [i for i in range(n) if i not in dead]
        e_f32 = errors(got[0, live], want[0, live])
        e_model = errors(want_rounded[0, live], want[0, live])
        print(f"  kernel vs fp32 oracle {e_f32}\n  rounded-operand oracle vs fp32 oracle {e_model}", flush=True)
        # operand rounding alone costs what the kernel is off by ...
        assert e_model["max_abs"] > 5 * 2e-2 and e_f32["max_abs"] < 1.5 * e_model["max_abs"]
        # ... and against the same arithmetic the kernel meets the unscaled limits
        print(assert_close(got[0, live], want_rounded[0, live], "rows with a valid key, large logits, "
                           "against the rounded-operand oracle"), flush=True)
        # fully masked rows: gate * mean of v over all N keys, projected
        v_mean = ref.mha.linear_v(xn[0, dead]).mean(dim=1, keepdim=True)           # [rows, 1, 128]
        gate = torch.sigmoid(ref.mha.linear_g(xn[0, dead]))                         # [rows, N, 128]
        uniform = ref.mha.linear_o(gate * v_mean)
        assert_close(got[0, dead], uniform, "fully masked rows attend uniformly", auto_scale=True)
        # the reference itself is far from uniform here (residues of 64): the stated deviation
        assert (want[0, dead] - uniform).abs().max() > 10 * (got[0, dead] - uniform).abs().max()
        # ... and agrees with the kernel once the logits are below 32: scale q down
        ref.mha.linear_q.weight.mul_(1e-3)
        ref.linear.weight.mul_(1e-2)
        hip.load_state_dict(ref.state_dict())
        got2 = hip(xb.to(DEV), mask.to(DEV)).float().cpu()
        want2 = ref(xb.float(), mask.float())
        assert_close(got2[0, dead], want2[0, dead], "fully masked rows, |logits| < 32", auto_scale=True)
        assert_close(want2[0, dead], uniform, "oracle is uniform there too", auto_scale=True,
                     max_abs=1e-4, mean_abs=1e-5, rel_fro=1e-4)
