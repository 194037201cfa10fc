"""The C-ABI library loads without a GPU and exports every symbol include/kfold_hip.h declares."""

import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


def _declared():
    text = (ROOT / "include" / "kfold_hip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(kfh_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_exported_and_bound():
    from kfold_amd import _lib

    names = _declared()
    assert len(names) >= 20
    lib = _lib.lib()                       # raises ImportError if the library is not built
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in kfold_hip.h but not exported"
    assert sorted(_lib.SIGNATURES) == names, "ctypes table and header disagree"
    assert lib.kfh_version() >= 1


def test_size_queries_and_argument_errors_need_no_gpu():
    from kfold_amd import _lib

    lib = _lib.lib()
    assert lib.kfh_trimul_packed_bytes(128) > 0 and lib.kfh_trimul_packed_bytes(64) == 0
    assert lib.kfh_trimul_packed_bytes(256) > lib.kfh_trimul_packed_bytes(128)
    assert lib.kfh_triattn_packed_bytes(128, 4) > 0 and lib.kfh_triattn_packed_bytes(128, 3) == 0
    assert lib.kfh_triattn_packed_bytes(64, 4) > 0 and lib.kfh_triattn_packed_bytes(128, 1) == 0   # head dim > 64
    # workspace grows with N and is 256-byte granular
    w1, w2 = lib.kfh_trimul_workspace_bytes(384, 128), lib.kfh_trimul_workspace_bytes(768, 128)
    assert 0 < w1 < w2 and w1 % 256 == 0
    assert lib.kfh_transition_workspace_bytes(1000, 128, 2) == 0       # fused pair kernel
    assert lib.kfh_transition_workspace_bytes(1000, 384, 4) > 0
    assert lib.kfh_apb_packed_bytes(384, 16, 0) > 0 and lib.kfh_apb_packed_bytes(384, 5, 0) == 0
    # argument checks run before any GPU call
    rc = lib.kfh_trimul_forward(None, None, None, None, None, None, 0, 1, 8, 64, 0, 1e-5, 0, None)
    assert rc == -2 and b"C=64" in lib.kfh_last_error()
    rc = lib.kfh_trimul_forward(None, None, None, None, None, None, 0, 1, 8, 128, 0, 1e-5, 0, None)
    assert rc == -1 and b"null" in lib.kfh_last_error()
    rc = lib.kfh_triattn_forward(None, None, None, None, None, None, 0, 1, 9000, 128, 4, 0, 1e-5, 0, None)
    assert rc == -2


def test_backend_selection_without_gpu():
    import kfold_amd

    assert kfold_amd.select_kernel_backend("torch") == "torch"
    with pytest.raises(ValueError):
        kfold_amd.select_kernel_backend("cuda")
    import torch
    if not torch.cuda.is_available():
        assert kfold_amd.select_kernel_backend("auto") == "torch"
        with pytest.raises(ValueError):
            kfold_amd.select_kernel_backend("hip")


def test_state_dict_names_match_reference_names():
    """Parameter names of the product modules are the reference's (and the oracle's)."""
    from kfold_amd import layers, modules, primitives
    from oracle import torch_path as O

    pairs = [
        (primitives.TriangleMultiplicationOutgoing(128), O.TriangleMultiplicationOutgoing(128)),
        (primitives.TriangleAttentionEndingNode(128, 4), O.TriangleAttentionEndingNode(128, 4)),
        (layers.Transition(128, 2), O.Transition(128, 2)),
        (layers.SelfAttentionPairBias(384, 16, None, "confidence"), O.SelfAttentionPairBias(384, 16, None)),
        (layers.SelfAttentionPairBias(768, 16, 384, "diffusion_global"),
         O.SelfAttentionPairBias(768, 16, 384, call_site="diffusion_global")),
        (modules.PairSingleBlock(), O.PairSingleBlock()),
    ]
    for hip, ref in pairs:
        a, b = hip.state_dict(), ref.state_dict()
        assert sorted(a) == sorted(b)
        assert all(a[k].shape == b[k].shape for k in a)
    tm = primitives.TriangleMultiplicationIncoming(128).state_dict()
    assert set(tm) == {"layernorm_in.weight", "layernorm_in.bias", "linear_p_in.weight",
                       "linear_g_in.weight", "layernorm_out.weight", "layernorm_out.bias",
                       "linear_p_out.weight", "linear_g_out.weight"}
    ta = primitives.TriangleAttentionStartingNode(128, 4).state_dict()
    assert set(ta) == {"layer_norm.weight", "layer_norm.bias", "linear.weight", "mha.linear_q.weight",
                       "mha.linear_k.weight", "mha.linear_v.weight", "mha.linear_o.weight",
                       "mha.linear_g.weight"}


def test_no_cpu_fallback_in_the_product_path():
    """The modules never compute on the host: CPU tensors are refused, training mode is refused,
    and nothing under kfold_amd imports the oracle."""
    import torch

    from kfold_amd import layers, primitives

    x = torch.zeros(1, 8, 8, 128)
    m = torch.ones(1, 8, 8)
    for mod in (primitives.TriangleMultiplicationOutgoing(128).eval(),
                primitives.TriangleAttentionStartingNode(128, 4).eval()):
        with pytest.raises((RuntimeError, ValueError)):
            with torch.no_grad():
                mod(x, m)
    with pytest.raises((RuntimeError, ValueError)):
        with torch.no_grad():
            layers.Transition(128, 2).eval()(x)
    for path in (ROOT / "kfold_amd").rglob("*.py"):
        text = path.read_text()
        assert "import oracle" not in text and "from oracle" not in text, path
    # the benchmark may only use the oracle for its cpu_baseline leg
    text = (ROOT / "bench.py").read_text()
    current = ""
    uses = 0
    for line in text.splitlines():
        if line.startswith("def "):
            current = line.split("(")[0][4:]
        if "from oracle" in line or "import oracle" in line:
            uses += 1
            assert current.startswith("cpu_baseline"), f"bench.py: oracle used in {current}()"
    assert uses >= 1
