#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X: one Pairformer block at N=768, bf16.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--n 768] [--no-cpu-baseline]

A step is one forward pass of one block (pair track: triangle multiplication out/in, triangle
attention start/end, transition, final mask; single track: pair bias from z, pair-bias
attention, transition) on synthetic z [1,N,N,128], s [1,N,384] with 12 % trailing token
padding and random-init weights (trunc-normal std 0.02), resident in HBM before the timed
region.  Prints ONE JSON line: the block time (the headline metric), per-op times, the
roofline position of the dominant kernel (timed live with events on the launch stream) and
the CPU oracle timed on the host cores as a baseline.
"""

from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0      # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0          # MI355X HBM3E
CAL_COPY_BYTES = 256 << 20     # size of the counter-calibration copy
# HBM bytes per launch of the attention kernel at N=768 (FETCH_SIZE + WRITE_SIZE, each scaled by
# the calibration copy's reading in the same run); the counter runs are summarised in
# profiles/hot_path_kernels_n768_hbm_traffic.md.  None where no counter run exists.
MEASURED_TRAFFIC_BYTES = {768: 851100477}


def block_flops(n: int) -> dict:
    """Algorithmic flops of one block (C = 128, tri-attn 4x32, single track 384 / 16x24)."""
    trimul = 256 * n**3 + 196608 * n**2
    triattn = 512 * n**3 + 164864 * n**2
    transition = 98304 * 2 * n**2
    cs, hs = 384, 16
    single = 2 * 128 * hs * n**2 + 10 * cs * cs * n + 4 * n * n * cs + 6 * cs * cs * 4 * n
    return {"trimul": trimul, "triattn": triattn, "transition": transition, "single": single,
            "block": 2 * trimul + 2 * triattn + transition + single}


def event_time_ms(fn, iters: int, warm: int = 2) -> list[float]:
    import torch

    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    out = []
    for _ in range(iters):
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        fn()
        e.record()
        e.synchronize()
        out.append(s.elapsed_time(e))
    return out


def cpu_baseline(n_sample: int, n_target: int) -> dict:
    """The fp32 oracle (a port of the reference's torch path) on the host cores: one block at
    n_sample tokens, timed once after a small warm-up call; when n_sample differs from the
    target N the time is scaled by the algorithmic flop count."""
    import torch

    from kfold_amd import synthetic
    from oracle import torch_path as O

    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    blk = O.PairSingleBlock(row_chunk=32).eval()
    synthetic.init_weights_(blk, 0)
    z, tok, pm = synthetic.pair_inputs(n_sample, 128, synthetic.n_pad_for(n_sample, 0.12), 0)
    s = synthetic.single_inputs(n_sample, 384, 1)
    with torch.inference_mode():
        blk(z[:, :32, :32].clone(), s[:, :32].clone(), pm[:, :32, :32].float(), tok[:, :32].float())
        t0 = time.perf_counter()
        blk(z.clone(), s.clone(), pm.float(), tok.float())
        dt = (time.perf_counter() - t0) * 1e3
    scale = block_flops(n_target)["block"] / block_flops(n_sample)["block"]
    direct = n_sample == n_target
    return {
        "value": round(dt * scale, 1),
        "unit": f"ms per Pairformer block at N={n_target}" + ("" if direct else " (extrapolated by flop count)"),
        "cores": cores,
        "kind": "port",
        "sample": (f"one whole block at N={n_sample}, fp32 torch oracle, one timed pass" if direct else
                   f"one block at N={n_sample}, fp32 torch oracle, measured {dt:.0f} ms; "
                   f"x{scale:.2f} flops to N={n_target}"),
    }


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--n", type=int, default=768, help="tokens (the metric is quoted at 768)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-sample-n", type=int, default=0,
                    help="tokens of the CPU baseline sample (0: the benchmark's own N, timed directly)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); "
              f"--gpus {args.gpus} is not supported", file=sys.stderr)
        return 2

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no ROCm GPU visible", file=sys.stderr)
        return 1
    from kfold_amd import _lib, modules, ops, synthetic

    _lib.lib()                                         # fail loudly if the library is not built
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    n = args.n
    n_pad = synthetic.n_pad_for(n, 0.12)
    block = modules.PairSingleBlock().eval()
    synthetic.init_weights_(block, 0)
    block.to(dev)
    z0, tok, pm = synthetic.pair_inputs(n, 128, n_pad, 0)
    s0 = synthetic.single_inputs(n, 384, 1)
    z = z0.to(torch.bfloat16).to(dev)
    s = s0.to(torch.bfloat16).to(dev)
    pm, tok = pm.to(dev), tok.to(dev)
    fl = block_flops(n)

    # One plain device copy of known size (256 MiB read + 256 MiB written).  It plays no part in
    # the timing; under `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` its counter reading gives the
    # scale factor of those counters for the `roofline.traffic` figure.
    cal_src = torch.empty(CAL_COPY_BYTES, dtype=torch.uint8, device=dev)
    cal_dst = torch.empty_like(cal_src)
    cal_dst.copy_(cal_src)
    torch.cuda.synchronize()
    del cal_src, cal_dst

    with torch.inference_mode():
        def step():
            block(z, s, pm, tok, inplace_output=True)

        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

        # ---- per-op times (fresh inputs so the values are those of the first block) ---------
        zb = z0.to(torch.bfloat16).to(dev)
        sb = s0.to(torch.bfloat16).to(dev)
        pb = block.pair_block
        from kfold_amd.layers.transition import hip_transition
        opfn = {
            "trimul_out": lambda: pb.tri_mul_out(zb, pm),
            "trimul_in": lambda: pb.tri_mul_in(zb, pm),
            "triattn_start": lambda: pb.tri_att_start(zb, pm),
            "triattn_end": lambda: pb.tri_att_end(zb, pm),
            "pair_transition": lambda: pb.transition_z(zb),
            "single_track": lambda: _single_track(block, zb, sb, tok),
        }
        opflops = {"trimul_out": fl["trimul"], "trimul_in": fl["trimul"], "triattn_start": fl["triattn"],
                   "triattn_end": fl["triattn"], "pair_transition": fl["transition"],
                   "single_track": fl["single"]}
        ops_ms = {}
        for name, fn in opfn.items():
            ms = statistics.median(event_time_ms(fn, 5))
            ops_ms[name] = {"ms": round(ms, 4), "tflops": round(opflops[name] / ms / 1e9, 1),
                            "mfma_frac": round(opflops[name] / ms / 1e9 / PEAK_BF16_TFLOPS, 4)}

        # ---- dominant kernel: the attention kernel of triangle attention, timed alone ---------
        L = _lib.lib()
        mod = pb.tri_att_start
        mod(zb, pm)                                     # builds the packed-weight cache
        blob = mod._hip_attention_cache
        ws_bytes = L.kfh_triattn_workspace_bytes(n, 128, 4)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        out = torch.empty_like(zb)
        m8 = pm.contiguous().view(torch.uint8)
        stream = torch.cuda.current_stream(dev).cuda_stream

        def stage(which):
            _lib.check(L.kfh_triattn_forward_stages(zb.data_ptr(), m8.data_ptr(), blob.data_ptr(), None,
                                                    out.data_ptr(), ws.data_ptr(), ws_bytes, 1, n, 128, 4,
                                                    0, 1e-5, _lib.KFH_BF16, which, stream))

        stage(_lib.KFH_STAGE_IN)
        flash_ms = event_time_ms(lambda: stage(_lib.KFH_STAGE_CORE), max(args.steps, 10))
        flash_avg = sum(flash_ms) / len(flash_ms)
        flash_flops = 512 * n**3                        # QK^T + PV, 4 heads x 32
        achieved = flash_flops / flash_avg / 1e9

    result = {
        "metric": f"ms per Pairformer block at N={n} bf16",
        "value": round(ms_per_step, 4),
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"pairformer_block_N{n}", "n_tokens": n, "n_padded_tokens": n_pad,
                   "c_z": 128, "c_s": 384, "tri_heads": "4x32", "apb_heads": "16x24",
                   "pair_transition_expansion": 2, "single_transition_expansion": 4},
        "block_tflops": round(fl["block"] / ms_per_step / 1e9, 1),
        "block_mfma_frac": round(fl["block"] / ms_per_step / 1e9 / PEAK_BF16_TFLOPS, 4),
        "ops": ops_ms,
        "roofline": {
            "kernel": "flash_strip_kernel (triangle attention, QK^T + softmax + PV)",
            "bound": "mfma",
            "achieved": round(achieved, 1),
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
            "traffic": MEASURED_TRAFFIC_BYTES.get(n),
            "avg_launch_ms": round(flash_avg, 4),
            "flops_per_launch": flash_flops,
        },
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(args.cpu_sample_n or n, n)
    print(json.dumps(result))
    return 0


def _single_track(block, z, s, tok):
    """The single-track part of the block alone: pair bias from z, attention, transition."""
    import torch

    from kfold_amd import ops
    from kfold_amd.layers.attention_pair_bias import _parameters
    from kfold_amd.layers.transition import hip_transition

    tiles = ops.pair_bias_project(z, block._hip_pair_bias_cache, block.num_heads)
    att = block.attention
    ops.apb_forward(s, None, tiles, tok.reshape(1, -1), att._hip_apb_cache, att.num_heads, 0, True, False,
                    residual=s, out=s)
    hip_transition(block.transition, s, residual=s, out=s)


if __name__ == "__main__":
    sys.exit(main())
