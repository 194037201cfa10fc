"""bench.py's helpers that no GPU is needed for: the counter-summary reader, and the shipping-width
rows of the configuration table run through the kernels' host build at small sizes (every module
call of those rows executes; the times are stand-ins)."""

import json
import math

import pytest


def test_traffic_rows_follow_the_built_machine_code(tmp_path, monkeypatch):
    import bench
    from kfold_amd.build import ISA_JSON

    if not ISA_JSON.exists():
        pytest.skip("library not built by kfold_amd.build")
    rows, why = bench.read_traffic_profile(768)
    assert why is None, why
    assert any(k.startswith("kfh::flash_strip_kernel") for k in rows)
    for rd, wr in rows.values():
        assert rd >= 0 and wr >= 0
    # another N: no rows, with the reason
    rows_n, why_n = bench.read_traffic_profile(512)
    assert rows_n == {} and "N=768" in why_n
    # a kernel whose machine code differs from the measured one loses its row
    built = json.loads(ISA_JSON.read_text())
    key = next(k for k in built if "flash_strip_kernel" in k)
    built[key] = "0" * 16
    other = tmp_path / "kernel_isa.json"
    other.write_text(json.dumps(built))
    import kfold_amd.build as kb

    monkeypatch.setattr(kb, "ISA_JSON", other)
    rows2, why2 = bench.read_traffic_profile(768)
    assert why2 is None and not any(k.startswith("kfh::flash_strip_kernel") for k in rows2)
    assert len(rows2) == len(rows) - 1
    other.write_text("{}")
    rows3, why3 = bench.read_traffic_profile(768)
    assert rows3 == {} and "other machine code" in why3


def test_shipping_width_rows_run_on_the_host_build():
    import torch

    import bench
    from tests import hostsim

    calls = []

    def time_ms(fn):
        fn()
        calls.append(1)
        return 1.0

    with hostsim.host_backend(), torch.no_grad():
        rows = bench.shipping_dim_rows(hostsim.HostDevice("cpu"), time_ms, n_wide=40, n_templates=36,
                                       n_atoms_windows=2, n_tokens=40)
    assert len(rows) == len(calls) == 7
    assert [r["config"] for r in rows] == ["F2"] * 5 + ["F3"] * 2
    for r in rows:
        assert r["hip_ms"] == 1.0 and isinstance(r["what"], str) and isinstance(r["roof"], str)
        assert r["tflops"] is None or (math.isfinite(r["tflops"]) and r["tflops"] > 0)
    json.dumps(rows)


def test_host_model_vectors_are_current():
    """tests/golden/host_model_vectors.pt is what the host build gives today, bit for bit (a kernel
    change that moves a result has to regenerate it: python -m tests.golden.make_host_model_vectors)."""
    from tests import hostsim
    from tests.test_zy_host_model_vectors_gpu import compare

    with hostsim.host_backend():
        stats = compare(hostsim.HostDevice("cpu"))
    assert all(frac == 1.0 for frac, _ in stats.values()), stats


def test_smoke_body_on_the_host_build(capsys):
    """What __graft_entry__.smoke() runs on cuda:0, run on the kernels' host build: the call sequence,
    the oracle comparison and its thresholds."""
    import __graft_entry__ as entry
    from tests import hostsim

    with hostsim.host_backend():
        entry._smoke_on(hostsim.HostDevice("cpu"))
    assert "smoke ok" in capsys.readouterr().out


def test_per_kernel_table_on_the_host_build(monkeypatch):
    """bench.py's harness (stage-selective launches of one block's kernels) and its per-kernel table at
    a small size on the host build; the times are stand-ins."""
    import bench
    from tests import hostsim

    monkeypatch.setattr(bench, "event_time_ms", lambda fn, iters, warm=2: [(fn(), 1.0)[1]] * 2)
    import torch

    with hostsim.host_backend(), torch.inference_mode():        # as bench.main() calls them
        h = bench.Harness(40, 0.12, dev=hostsim.HostDevice("cpu"))
        assert h.flash_ms(2) == 1.0
        table = bench.per_kernel_table(h, {"kfh::flash_strip_kernel": (10.0, 5.0)}, iters=2)
    assert set(table) == {"trimul_in_kernel", "contract_kernel", "trimul_out_kernel", "triattn_proj_kernel",
                          "flash_strip_kernel", "triattn_out_kernel", "transition_kernel", "pair_bias_kernel"}
    assert table["flash_strip_kernel"]["measured_MB"] == 15.0 and table["contract_kernel"]["measured_MB"] is None
    assert bench.flash_executed_flops(h.pm, 40) > 0
    assert bench.block_flops(768)["block"] > 1.2e12
