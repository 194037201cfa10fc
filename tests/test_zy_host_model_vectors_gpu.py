"""The GPU's results against the results of the kernels' host build (tests/hostsim) on the same
calls: tests/golden/host_model_vectors.pt holds what the host build gives for a few small cases of
every operator family (written by tests/golden/make_host_model_vectors.py).  Host build and GPU round
to bf16 in the same places and differ only in the last bits of exp2 / rsqrt / reciprocal and in the
order of the fp32 sums inside an MFMA, so nearly all output values agree bit for bit; the fraction is
printed per case.  This ties what the host build verifies (every parity test, the address walks, the
random cases) to what the hardware executes."""

from pathlib import Path

import pytest
import torch

from tests.golden.make_host_model_vectors import cases
from tests.util import ulp_bf16

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
VECTORS = Path(__file__).resolve().parent / "golden" / "host_model_vectors.pt"
MIN_IDENTICAL = 0.9          # expected: > 0.999 (see the module docstring)


def compare(dev) -> dict:
    """{case: (fraction of bit-identical values, largest difference in units of the value's bf16
    spacing, or of 1e-6 relative for fp32 outputs)} for the device ``dev``."""
    want = torch.load(VECTORS, weights_only=True)
    stats = {}
    with torch.no_grad():
        for name, (build, inputs, call) in cases().items():
            mod = build().to(dev)
            got = call(mod, {k: v.to(dev) for k, v in inputs.items()}).detach().cpu()
            ref = want[name]
            assert got.shape == ref.shape and got.dtype == ref.dtype, name
            assert torch.isfinite(got.float()).all(), name
            same = (got.view(torch.int16 if got.dtype == torch.bfloat16 else torch.int32)
                    == ref.view(torch.int16 if ref.dtype == torch.bfloat16 else torch.int32))
            d = (got.float() - ref.float()).abs()
            # values close to zero are sums of far larger terms: their spacing is taken at 1/16 of the
            # tensor's RMS at least
            floor = ref.float().pow(2).mean().sqrt() / 16
            mag = ref.float().abs().clamp_min(floor)
            unit = ulp_bf16(mag) if got.dtype == torch.bfloat16 else mag * 1e-6
            stats[name] = (same.float().mean().item(), (d / unit).max().item())
    return stats


def test_gpu_results_against_the_host_builds():
    stats = compare(DEV)
    for name, (frac, worst) in stats.items():
        print(f"case {name}: {100 * frac:.3f} % of the values bit-identical to the host build, "
              f"largest difference {worst:.2f} units", flush=True)
    for name, (frac, worst) in stats.items():
        if name.endswith("_f32"):
            assert worst <= 200, (name, frac, worst)          # 2e-4 of the value: fp32 arithmetic on both sides
        else:
            assert frac >= MIN_IDENTICAL, (name, frac, worst)
            assert worst <= 16, (name, frac, worst)           # a few bf16 steps at most
