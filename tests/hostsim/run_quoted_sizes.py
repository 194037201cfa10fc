"""Run the quoted-size parity cases of tests/test_quoted_sizes_gpu.py (and the other cases the unit
suite leaves out for CPU time) on the host execution model:

    python -m tests.hostsim.run_quoted_sizes [substring of a test name ...]

Minutes to an hour of CPU time per case, which is why pytest does not collect this file.  The 48-block
trunk is left to the GPU (48 blocks at N = 1024 are hours here); its single blocks are covered by
the N = 1024 cases.
"""

from __future__ import annotations

import sys
import time

import tests.test_zx_row_ranges_gpu as BK
import tests.test_quoted_sizes_gpu as Q
import tests.test_shipping_dims_gpu as SD
import tests.test_triattn_gpu as TA
from tests import hostsim
from tests.test_hostsim_parity import _on_host

CASES = [
    (Q, "test_trimul_n768", [("outgoing",), ("incoming",)]),
    (Q, "test_triattn_n768_n1024_sampled_rows", [(768, 0.12, True), (768, 0.12, False),
                                                  (1024, 0.15, True), (1024, 0.15, False)]),
    (Q, "test_apb_trunk_variant_n768", [()]),
    (Q, "test_apb_diffusion_variant_n768", [(False,), (True,)]),
    (Q, "test_block_n768_metric_shape", [()]),
    (TA, "test_triattn_long_sequence_sampled_rows", [()]),
    (TA, "test_triattn_config3_n512", [(True,), (False,)]),
    (SD, "test_triattn_c64_templates_n384", [(True,), (False,)]),
    (SD, "test_trimul_c256_tiled_sizes", [("outgoing", 384), ("incoming", 384), ("outgoing", 768), ("incoming", 768)]),
    (BK, "test_phases_over_row_ranges_at_the_benchmark_size", [()]),
]


def main(argv: list[str]) -> int:
    failed = 0
    for mod, name, params in CASES:
        if argv and not any(a in name for a in argv):
            continue
        for p in params:
            t0 = time.time()
            print(f"=== {name}{p}", flush=True)
            try:
                with _on_host(mod):
                    getattr(mod, name)(*p)
                print(f"=== PASSED {name}{p} in {time.time() - t0:.0f} s", flush=True)
            except Exception as e:  # noqa: BLE001
                failed += 1
                print(f"=== FAILED {name}{p}: {type(e).__name__}: {e}", flush=True)
    hostsim.load().hostsim_report()
    return 1 if failed else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
