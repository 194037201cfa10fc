"""Every kernel launch that the host build has seen in this process (this file sorts after the other
host-build tests, and runs a small workload of its own) against the compiler's record of the gfx950
kernels: a workgroup larger than the kernel's ``__launch_bounds__`` is refused by the GPU at launch,
which the host build by itself would not notice."""

import ctypes
import json
import re

import pytest
import torch

from kfold_amd import modules, synthetic
from tests import hostsim


def _launched() -> dict[str, int]:
    hs = hostsim.load()
    need = hs.hostsim_launch_shapes(None, 0)
    buf = ctypes.create_string_buffer(need)
    hs.hostsim_launch_shapes(buf, need)
    out: dict[str, int] = {}
    for line in buf.value.decode().splitlines():
        name, threads = line.rsplit("\t", 1)
        base = re.search(r"([A-Za-z_]\w*)\s*(<|\)|$)", name.replace("kfh::", "")).group(1)
        out[base] = max(out.get(base, 0), int(threads))
    return out


def test_launched_workgroups_fit_the_kernels_launch_bounds():
    from kfold_amd.build import RESOURCES_JSON

    if not RESOURCES_JSON.exists():
        pytest.skip("library not built by kfold_amd.build")
    resources = json.loads(RESOURCES_JSON.read_text())
    dev = hostsim.HostDevice("cpu")
    with hostsim.host_backend(), torch.no_grad():
        n = 40
        z, tok, pm = synthetic.pair_inputs(n, 128, 5, 0)
        blk = modules.PairSingleBlock().eval()
        synthetic.init_weights_(blk, 0)
        blk.to(dev)
        blk(z.bfloat16().to(dev), synthetic.single_inputs(n, 384, 1).bfloat16().to(dev), pm.to(dev), tok.to(dev))
        wide = modules.TriangularBlock(256).eval()
        synthetic.init_weights_(wide, 1)
        wide.to(dev)
        wide(torch.randn(1, n, n, 256).bfloat16().to(dev), pm.to(dev))
    launched = _launched()
    assert len(launched) >= 10, launched
    for base, threads in launched.items():
        tag = f"{len(base)}{base}"
        bounds = [r["max_flat_workgroup_size"] for name, r in resources.items() if tag in name]
        assert bounds, f"kernel {base} was launched on the host build but is not in the gfx950 library"
        assert threads <= min(bounds), f"{base}: launched with {threads} threads, built for {min(bounds)}"
