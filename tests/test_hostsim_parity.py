"""The GPU parity tests, run on the CPU through the host execution model of the kernels.

Every ``test_*`` function of the ``*_gpu`` test modules gets a twin here that runs the same body
with ``DEV = "cpu"`` while ``tests.hostsim.host_backend()`` routes the product's Python layer to
``libkfold_hostsim.so`` — the kernel sources themselves, compiled for the host, lanes as fibers,
MFMA / shuffles / barriers as rendezvous, workspaces between guard pages and pre-filled with NaN.
So module → functional layer → C ABI → kernel code is compared with the oracle exactly as on the
GPU, minus what only hardware can show (timing, memory-ordering between lanes of a wavefront).

Cases that need a device (streams, CPU-tensor rejection) or more CPU time than a unit suite
should take are listed in ``SKIP`` with the reason; the big ones carry the ``slow`` marker's
twin in ``tests/hostsim/run_quoted_sizes.py`` instead.
"""

from __future__ import annotations

import contextlib
import functools
import importlib

import pytest
import torch

from tests import hostsim

GPU_MODULES = [
    "tests.test_trimul_gpu",
    "tests.test_triattn_gpu",
    "tests.test_single_track_gpu",
    "tests.test_block_gpu",
    "tests.test_shipping_dims_gpu",
    "tests.test_parcae_gpu",
    "tests.test_zx_row_ranges_gpu",
    "tests.test_zy_host_model_vectors_gpu",
    "tests.test_zz_no_alloc",
]

# test name (or "name[param id]") -> reason it has no CPU twin
SKIP: dict[str, str] = {
    "test_phases_over_row_ranges_at_the_benchmark_size": "N = 768: minutes of CPU time "
                                                         "(tests/hostsim/run_quoted_sizes.py runs it; N = 260 stays here)",
    "test_cpu_tensors_are_rejected": "the twin runs on CPU tensors by design",
    "test_triattn_long_sequence_sampled_rows": "N = 1248 takes two minutes of CPU time "
                                               "(tests/hostsim/run_quoted_sizes.py runs it)",
    "test_triattn_config3_n512": "benchmark config 3 at N = 512: a quarter of a minute of CPU time per node type "
                                 "(tests/hostsim/run_quoted_sizes.py runs it; N = 256 and 130 stay here)",
    "test_triattn_c64_templates_n384": "4 templates at N = 384: half a minute of CPU time each "
                                       "(tests/hostsim/run_quoted_sizes.py runs them)",
    "test_trimul_c256_tiled_sizes": "N = 384 / 768 at C = 256: half a minute to minutes of CPU time each "
                                    "(tests/hostsim/run_quoted_sizes.py runs them)",
}


@contextlib.contextmanager
def _on_host(mod):
    saved = mod.DEV
    mod.DEV = hostsim.HostDevice("cpu")
    try:
        with hostsim.host_backend():
            yield
    finally:
        mod.DEV = saved


def _twin(mod, fn):
    @functools.wraps(fn)
    def run(*args, **kwargs):
        with _on_host(mod):
            return fn(*args, **kwargs)
    return run


for _name in GPU_MODULES:
    _mod = importlib.import_module(_name)
    _short = _name.rsplit(".", 1)[1].replace("test_", "").replace("_gpu", "")
    for _attr, _fn in list(vars(_mod).items()):
        if _attr.startswith("test_") and callable(_fn) and _attr not in SKIP:
            globals()[f"test_host_{_short}__{_attr[5:]}"] = _twin(_mod, _fn)


# The token-track linears pick between two kernels by problem size (one 32 x 32 tile per workgroup
# with K split over its wavefronts, or 128 x 128 tiles): the unit-sized cases above mostly take the
# first, so a selection of them runs again with the tile kernel forced wherever it applies.
import tests.test_shipping_dims_gpu as _SD      # noqa: E402
import tests.test_single_track_gpu as _ST       # noqa: E402

_TILE_CASES = [
    (_ST, "test_transition_parity", (384, 4, 70, torch.bfloat16)),
    (_ST, "test_pair_bias_projection_and_trunk_apb", (96,)),
    (_ST, "test_apb_functional_normalised_inputs_and_full_mask", ()),
    (_ST, "test_apb_diffusion_variant", (False,)),
    (_ST, "test_cross_attention_local_windows", (True,)),
    (_SD, "test_triattn_other_widths_batched", (True, 64, 4, 50, 4)),
    (_SD, "test_triattn_other_widths_batched", (False, 96, 2, 37, 2)),
    (_SD, "test_trimul_other_widths", ("incoming", 64, 70, 0)),
    (_SD, "test_template_stack_block_c64", (torch.float32,)),
]


@pytest.mark.parametrize("mod,name,args", _TILE_CASES, ids=[f"{n}{list(a)}" for _, n, a in _TILE_CASES])
def test_host_tile_kernel_forced(mod, name, args, monkeypatch):
    monkeypatch.setenv("KFH_LINEAR_TILE_MIN_WORKGROUPS", "1")
    with _on_host(mod):
        getattr(mod, name)(*args)
