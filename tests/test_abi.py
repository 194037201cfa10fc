"""The C-ABI library loads without a GPU and exports every symbol include/kfold_hip.h declares."""

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
    assert lib.kfh_trimul_packed_bytes(128) > 0 and lib.kfh_trimul_packed_bytes(64) > 0 and lib.kfh_trimul_packed_bytes(48) == 0
    assert lib.kfh_trimul_packed_bytes(256) > lib.kfh_trimul_packed_bytes(128)
    assert lib.kfh_triattn_packed_bytes(128, 4) > 0 and lib.kfh_triattn_packed_bytes(128, 3) == 0
    assert lib.kfh_triattn_packed_bytes(64, 4) > 0 and lib.kfh_triattn_packed_bytes(128, 1) == 0   # head dim > 64
    # workspace grows with N and is 256-byte granular
    w1, w2 = lib.kfh_trimul_workspace_bytes(384, 128), lib.kfh_trimul_workspace_bytes(768, 128)
    assert 0 < w1 < w2 and w1 % 256 == 0
    # batched sizes: the fused widths run batch elements in turn, the assembled ones can fold them
    assert lib.kfh_trimul_workspace_bytes_batched(4, 384, 128) == w1
    assert lib.kfh_trimul_workspace_bytes_batched(1, 100, 64) == lib.kfh_trimul_workspace_bytes(100, 64)
    assert lib.kfh_trimul_workspace_bytes_batched(4, 100, 64) > 3 * lib.kfh_trimul_workspace_bytes(100, 64)
    assert lib.kfh_triattn_workspace_bytes_batched(4, 100, 128, 4) == lib.kfh_triattn_workspace_bytes(100, 128, 4)
    assert lib.kfh_triattn_workspace_bytes_batched(4, 100, 64, 4) > 3 * lib.kfh_triattn_workspace_bytes(100, 64, 4)
    assert lib.kfh_trimul_workspace_bytes_batched(0, 100, 64) == 0 and lib.kfh_triattn_workspace_bytes_batched(4, 100, 48, 4) == 0
    assert lib.kfh_transition_workspace_bytes(1000, 128, 2) == 0       # fused pair kernel
    assert lib.kfh_transition_workspace_bytes(1000, 384, 4) > 0
    assert lib.kfh_apb_packed_bytes(384, 16, 0, 0) > 0 and lib.kfh_apb_packed_bytes(384, 5, 0, 0) == 0
    # argument checks run before any GPU call
    rc = lib.kfh_trimul_forward(None, None, None, None, None, None, 0, 1, 8, 48, 0, 1e-5, 0, None)
    assert rc == -2 and b"C=48" in lib.kfh_last_error()
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


def test_trunk_and_window_modules_keep_reference_names():
    """State-dict keys of the trunk-level and local-window modules, spelled out from the reference's
    attribute names (modules/tri_stack.py:31-151, model/model.py:201-217,
    layers/folding/attention_pair_bias.py:161-204), and equal to the oracle's."""
    from kfold_amd import layers, modules
    from oracle import torch_path as O

    pairs = [
        (modules.TriangularBlock(256), O.TriangularBlock(256)),
        (modules.TrianglularStack(256, 2), O.TrianglularStack(256, 2)),
        (modules.ParcaeStep(128), O.ParcaeStep(128)),
        (modules.ParcaeTrunk(128, lm_blocks=1, main_blocks=2), O.ParcaeTrunk(128, lm_blocks=1, main_blocks=2)),
        (layers.CrossAttentionPairBias(128, 4, None), O.CrossAttentionPairBias(128, 4, None)),
        (layers.CrossAttentionPairBias(128, 4, 64), O.CrossAttentionPairBias(128, 4, 64)),
    ]
    for hip, ref in pairs:
        a, b = hip.state_dict(), ref.state_dict()
        assert sorted(a) == sorted(b), type(hip).__name__
        assert all(a[k].shape == b[k].shape for k in a), type(hip).__name__
    blk = set(modules.TriangularBlock(256).state_dict())
    assert {"tri_mul_out.linear_p_in.weight", "tri_mul_in.linear_g_out.weight",
            "transition_z.swiglu.linear.weight", "transition_z.linear_out.weight"} <= blk
    assert not any(k.startswith("tri_att") for k in blk)
    trunk = set(modules.ParcaeTrunk(128, lm_blocks=1, main_blocks=2).state_dict())
    assert {"parcae_log_a", "parcae_log_delta", "parcae_b_cont", "layernorm_z.weight",
            "lm_stack.blocks.0.tri_mul_out.layernorm_in.weight",
            "main_stack.blocks.1.transition_z.layernorm.weight"} <= trunk
    win = set(layers.CrossAttentionPairBias(128, 4, 64).state_dict())
    assert {"adaln_a_q.linear_g.weight", "adaln_a_k.linear_bias.weight", "linear_ada_out.bias",
            "linear_q.bias", "linear_out.weight"} <= win and "linear_k.bias" not in win
    plain = set(layers.CrossAttentionPairBias(128, 4, None).state_dict())
    assert {"layernorm_a_q.weight", "layernorm_a_k.bias"} <= plain and "linear_ada_out.weight" not in plain


def test_load_reference_weights_by_prefix():
    """Loading goes by the reference's names below a prefix, ignores the rest of a checkpoint, and
    refuses missing entries and wrong shapes."""
    import torch

    from kfold_amd import modules
    from kfold_amd.runtime import load_reference_weights
    from oracle import torch_path as O

    torch.manual_seed(0)
    ref = O.ParcaeTrunk(128, lm_blocks=1, main_blocks=2)
    with torch.no_grad():
        for p in ref.parameters():
            p.copy_(torch.randn_like(p))
    ckpt = {"trunk." + k: v for k, v in ref.state_dict().items()}
    ckpt["distogram_head.weight"] = torch.zeros(3)               # something without a hip counterpart
    hip = modules.ParcaeTrunk(128, lm_blocks=1, main_blocks=2)
    used = load_reference_weights(hip, ckpt, prefix="trunk.")
    assert sorted(used) == sorted(k for k in ckpt if k.startswith("trunk."))
    for k, v in hip.state_dict().items():
        assert torch.equal(v, ckpt["trunk." + k]), k
    # one stack out of the same checkpoint
    stack = modules.TrianglularStack(128, 2)
    load_reference_weights(stack, ckpt, prefix="trunk.main_stack.")
    assert torch.equal(stack.blocks[1].tri_mul_in.linear_p_in.weight,
                       ckpt["trunk.main_stack.blocks.1.tri_mul_in.linear_p_in.weight"])
    # a missing entry is an error unless strict is off; a wrong shape always is
    short = dict(ckpt)
    del short["trunk.parcae_log_a"]
    with pytest.raises(KeyError, match="parcae_log_a"):
        load_reference_weights(modules.ParcaeTrunk(128, lm_blocks=1, main_blocks=2), short, prefix="trunk.")
    partial = modules.ParcaeTrunk(128, lm_blocks=1, main_blocks=2)
    before = partial.parcae_log_a.detach().clone()
    used = load_reference_weights(partial, short, prefix="trunk.", strict=False)
    assert "trunk.parcae_log_a" not in used and torch.equal(partial.parcae_log_a, before)
    bad = dict(ckpt)
    bad["trunk.parcae_b_cont"] = torch.zeros(64, 64)
    with pytest.raises(ValueError, match="parcae_b_cont"):
        load_reference_weights(modules.ParcaeTrunk(128, lm_blocks=1, main_blocks=2), bad, prefix="trunk.")


def test_recurrence_window_and_static_entry_points_check_arguments_without_gpu():
    from kfold_amd import _lib

    lib = _lib.lib()
    assert lib.kfh_parcae_packed_bytes(128) > 0 and lib.kfh_parcae_packed_bytes(256) > lib.kfh_parcae_packed_bytes(128)
    assert lib.kfh_parcae_packed_bytes(64) == 0 and lib.kfh_parcae_packed_bytes(384) == 0
    rc = lib.kfh_parcae_step(None, None, None, None, None, 10, 64, 1e-5, 0, None)
    assert rc == -2, lib.kfh_last_error()
    rc = lib.kfh_parcae_step(None, None, None, None, None, 10, 128, 1e-5, 0, None)
    assert rc == -1, lib.kfh_last_error()
    # local attention windows: channels a multiple of 32, head dim at most 64
    assert lib.kfh_cross_apb_packed_bytes(128, 4, 0, 0) > 0 and lib.kfh_cross_apb_packed_bytes(128, 4, 64, 0) > lib.kfh_cross_apb_packed_bytes(128, 4, 0, 0)
    assert lib.kfh_cross_apb_packed_bytes(128, 1, 0, 0) == 0 and lib.kfh_cross_apb_packed_bytes(100, 4, 0, 0) == 0
    w1 = lib.kfh_cross_apb_workspace_bytes(10, 32, 128, 128, 4, 0, 0)
    w2 = lib.kfh_cross_apb_workspace_bytes(20, 32, 128, 128, 4, 0, 0)
    assert 0 < w1 < w2
    # allocation-free transition: 8 MiB of static scratch; a request beyond it is refused before
    # anything touches the GPU, with the limit in the message
    cap = lib.kfh_transition_static_scratch_bytes()
    assert cap == 8 << 20
    rows_ok, rows_big = 2184, 2185
    assert lib.kfh_transition_workspace_bytes(rows_ok, 384, 4) <= cap < lib.kfh_transition_workspace_bytes(rows_big, 384, 4)
    rc = lib.kfh_transition_forward_static(None, None, None, None, None, rows_big, 384, 4, 1e-5, 0, None)
    assert rc == -1 and b"static" in lib.kfh_last_error() and str(cap).encode() in lib.kfh_last_error()
    rc = lib.kfh_transition_forward_static(None, None, None, None, None, -1, 384, 4, 1e-5, 0, None)
    assert rc == -1
    rc = lib.kfh_transition_forward_static(None, None, None, None, None, 10, 100, 4, 1e-5, 0, None)
    assert rc == -2


def test_header_is_plain_c_and_a_c_caller_links(tmp_path):
    """The boundary is a C ABI: the header compiles as strict C99 and a C program that includes it
    links against the library and gets the documented status codes (no GPU needed for these calls)."""
    import shutil
    import subprocess

    if shutil.which("gcc") is None:
        pytest.skip("gcc not found")
    lib_dir = ROOT / "kfold_amd"
    if not (lib_dir / "libkfold_hip.so").exists():
        pytest.fail("kfold_amd/libkfold_hip.so is not built")
    src = tmp_path / "caller.c"
    src.write_text(r'''
#include "kfold_hip.h"
#include <stdio.h>
#include <string.h>
int main(void) {
    if (kfh_version() < 1) return 1;
    if (kfh_trimul_packed_bytes(128) == 0 || kfh_trimul_packed_bytes(48) != 0) return 2;
    if (kfh_transition_static_scratch_bytes() != (size_t)8 << 20) return 3;
    int rc = kfh_trimul_forward(0, 0, 0, 0, 0, 0, 0, 1, 8, 48, KFH_OUTGOING, 1e-5f, KFH_BF16, 0);
    if (rc != KFH_EUNSUPPORTED || !strstr(kfh_last_error(), "C=48")) return 4;
    rc = kfh_trimul_forward(0, 0, 0, 0, 0, 0, 0, 1, 8, 128, KFH_OUTGOING, 1e-5f, KFH_BF16, 0);
    if (rc != KFH_EINVAL) return 5;
    /* a whole block from C: sizes, then the two calls (refused here: null pointers) */
    if (kfh_pair_block_workspace_bytes(1, 64, 128, 4, 2) == 0) return 6;
    if (kfh_single_track_workspace_bytes(1, 64, 128, 384, 16, 4) == 0) return 7;
    rc = kfh_pair_block_forward(0, 0, 0, 0, 0, 0, 0, 0, 0, 1, 64, 128, 4, 2, 1e-5f, KFH_BF16, 0);
    if (rc != KFH_EINVAL || !strstr(kfh_last_error(), "null")) return 8;
    rc = kfh_single_track_forward(0, 0, 0, 0, 0, 0, 0, 0, 1, 64, 128, 384, 16, 4, 1e-5f, KFH_BF16, 0);
    if (rc != KFH_EINVAL || !strstr(kfh_last_error(), "null")) return 9;
    if (kfh_trimul_row_granule(768, 128) != 256) return 10;
    printf("ok\n");
    return 0;
}
''')
    exe = tmp_path / "caller"
    cmd = ["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", f"-I{ROOT / 'include'}", str(src),
           "-o", str(exe), f"-L{lib_dir}", "-l:libkfold_hip.so", f"-Wl,-rpath,{lib_dir}"]
    done = subprocess.run(cmd, capture_output=True, text=True)
    assert done.returncode == 0, done.stderr
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert run.returncode == 0 and run.stdout.strip() == "ok", (run.returncode, run.stdout, run.stderr)
