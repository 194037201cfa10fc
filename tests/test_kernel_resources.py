"""What the compiler reports for every gfx950 kernel of the library (kfold_amd/kernel_resources.json,
written by the build): limits a launch would otherwise only meet on the GPU."""

import json

import pytest

LDS_PER_WORKGROUP = 160 * 1024        # gfx950: 160 KiB of LDS per compute unit
REGISTERS_PER_LANE = 512              # unified VGPR + AGPR file per lane

# kernels known to keep a few registers in scratch memory (bytes per lane); a new entry here is a
# decision, not an accident
SCRATCH_ALLOWED = {"flash_strip_kernel": 80, "trimul_out_kernel": 64}


@pytest.fixture(scope="module")
def resources():
    from kfold_amd.build import RESOURCES_JSON

    if not RESOURCES_JSON.exists():
        pytest.skip("library not built by kfold_amd.build")
    return json.loads(RESOURCES_JSON.read_text())


def test_every_kernel_fits_the_compute_unit(resources):
    assert len(resources) >= 60
    for name, r in resources.items():
        assert r["group_segment_fixed_size"] <= LDS_PER_WORKGROUP, (name, r)
        # vgpr_count is the unified total: it includes the accumulation registers
        assert r["agpr_count"] <= r["vgpr_count"] <= REGISTERS_PER_LANE, (name, r)
        # one workgroup of the declared size must fit the register file: 512 registers x 64 lanes x
        # 4 SIMDs hold (2048 / registers per lane) wavefronts of 64
        regs = max(r["vgpr_count"], 1)
        waves_that_fit = 4 * (REGISTERS_PER_LANE // ((regs + 7) // 8 * 8))
        assert r["max_flat_workgroup_size"] <= 64 * waves_that_fit, (name, r)


def test_scratch_memory_only_where_it_is_known(resources):
    for name, r in resources.items():
        allowed = max((v for k, v in SCRATCH_ALLOWED.items() if k in name), default=0)
        assert r["private_segment_fixed_size"] <= allowed, (
            f"{name}: {r['private_segment_fixed_size']} bytes of scratch per lane "
            f"({r['vgpr_spill_count']} spilled registers)")
