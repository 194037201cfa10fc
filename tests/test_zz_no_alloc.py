"""The allocation-free transition entry point (static device scratch) against the
workspace-taking one, through the C ABI."""

import pytest
import torch

from kfold_amd import synthetic

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _setup(C, E, seed):
    from kfold_amd import ops
    from kfold_amd.layers import Transition
    from kfold_amd.layers.transition import _parameters

    mod = Transition(C, E).eval()
    synthetic.init_weights_(mod, seed, std=0.05)
    mod.to(DEV)
    return ops.transition_pack(*_parameters(mod), device=torch.device(DEV))


def _both(blob, x, C, E, residual):
    """(out of kfh_transition_forward, out of kfh_transition_forward_static) for the same input."""
    from kfold_amd import _lib

    L = _lib.lib()
    rows = x.shape[0]
    stream = torch.cuda.current_stream().cuda_stream
    io = _lib.KFH_BF16 if x.dtype == torch.bfloat16 else _lib.KFH_F32
    res = x if residual else None
    want = torch.empty_like(x)
    ws_bytes = L.kfh_transition_workspace_bytes(rows, C, E)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=DEV)
    _lib.check(L.kfh_transition_forward(x.data_ptr(), blob.data_ptr(), None if res is None else res.data_ptr(),
                                        None, want.data_ptr(), ws.data_ptr(), ws_bytes, rows, C, E, 1e-5, io,
                                        stream))
    got = torch.full_like(x, float("nan"))
    _lib.check(L.kfh_transition_forward_static(x.data_ptr(), blob.data_ptr(),
                                               None if res is None else res.data_ptr(), None, got.data_ptr(),
                                               rows, C, E, 1e-5, io, stream))
    torch.cuda.synchronize()
    return want, got


def test_static_transition_matches_workspace_variant_twice_in_a_row():
    from kfold_amd import _lib
    from oracle import torch_path as O

    print("case no-alloc transition", flush=True)
    L = _lib.lib()
    assert L.kfh_transition_static_scratch_bytes() == 8 << 20
    C, E = 384, 4
    blob = _setup(C, E, 3)
    g = torch.Generator().manual_seed(5)
    # first call: a large input (N = 1024 tokens); second call: a smaller one, which finds the
    # first call's values in the shared scratch
    for rows, dtype, residual in [(1024, torch.bfloat16, True), (333, torch.bfloat16, False),
                                  (70, torch.float32, True)]:
        print(f"  rows={rows} {dtype} residual={residual}", flush=True)
        x = torch.randn(rows, C, generator=g).to(dtype).to(DEV)
        want, got = _both(blob, x, C, E, residual)
        assert torch.isfinite(got).all()
        assert torch.equal(got, want), "static-scratch result differs from the workspace variant"
    # and against the oracle, like any other entry point
    ref = O.Transition(C, E).eval()
    synthetic.init_weights_(ref, 3, std=0.05)
    x = torch.randn(200, C, generator=g).bfloat16()
    _, got = _both(blob, x.to(DEV), C, E, False)
    with torch.no_grad():
        want = ref(x.float())
    from tests.util import assert_close
    assert_close(got, want, "static transition vs oracle", auto_scale=True)
    # the fused pair kernel (C = 128) needs no scratch and passes through
    blob128 = _setup(128, 2, 4)
    x = torch.randn(500, 128, generator=g).bfloat16().to(DEV)
    want, got = _both(blob128, x, 128, 2, True)
    assert torch.equal(got, want)


def test_static_transition_rejects_what_does_not_fit():
    from kfold_amd import _lib

    L = _lib.lib()
    C, E = 384, 4
    blob = _setup(C, E, 3)
    rows = 2185                                    # 2184 rows is the most that fit in 8 MiB
    assert L.kfh_transition_workspace_bytes(rows, C, E) > L.kfh_transition_static_scratch_bytes()
    assert L.kfh_transition_workspace_bytes(rows - 1, C, E) <= L.kfh_transition_static_scratch_bytes()
    x = torch.zeros(rows, C, dtype=torch.bfloat16, device=DEV)
    out = torch.empty_like(x)
    rc = L.kfh_transition_forward_static(x.data_ptr(), blob.data_ptr(), None, None, out.data_ptr(), rows, C, E,
                                         1e-5, _lib.KFH_BF16, None)
    assert rc == -1 and b"static" in L.kfh_last_error()
    rc = L.kfh_transition_forward_static(x.data_ptr(), blob.data_ptr(), None, None, out.data_ptr(), rows - 1, C,
                                         E, 1e-5, _lib.KFH_BF16, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
