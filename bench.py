#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X: one Pairformer block at N=768, bf16.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--n 768] [--no-cpu-baseline]
                    [--no-extras] [--table]

A step is one forward pass of one block (pair track: triangle multiplication out/in, triangle
attention start/end, transition, final mask; single track: pair bias from z, pair-bias
attention, transition) on synthetic z [1,N,N,128], s [1,N,384] with 12 % trailing token
padding and random-init weights (trunc-normal std 0.02), resident in HBM before the timed
region.  Steps feed their output into the next step, as the blocks of a trunk do.

Prints ONE JSON line: the block time (the headline metric), per-op and per-kernel times, the
roofline position of the dominant kernel (timed live with events on the launch stream), the
48-block N=1024 trunk time, and the CPU oracle timed on the host cores as a baseline.
``--table`` additionally measures every benchmark configuration (C1..C5) and prints a markdown
table on stderr.
"""

from __future__ import annotations

import argparse
import hashlib
import json
import os
import re
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0      # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0          # MI355X HBM3E
CAL_COPY_BYTES = 256 << 20     # size of the counter-calibration copy
# rocprofv3 FETCH_SIZE / WRITE_SIZE summary of this very command; bench.py only reads it
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "hot_path_kernels_n768_hbm_traffic.txt")


def block_flops(n: int) -> dict:
    """Algorithmic flops of one block (C = 128, tri-attn 4x32, single track 384 / 16x24)."""
    trimul = 256 * n**3 + 196608 * n**2
    triattn = 512 * n**3 + 164864 * n**2
    transition = 98304 * 2 * n**2
    cs, hs = 384, 16
    single = 2 * 128 * hs * n**2 + 10 * cs * cs * n + 4 * n * n * cs + 6 * cs * cs * 4 * n
    return {"trimul": trimul, "triattn": triattn, "transition": transition, "single": single,
            "block": 2 * trimul + 2 * triattn + transition + single}


def kernel_sources_digest() -> str:
    """sha256 over the HIP sources: a traffic profile taken from other kernels is stale."""
    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "kfold_amd", "csrc")
    for name in sorted(os.listdir(csrc)):
        if name.endswith((".hip", ".hpp")):
            with open(os.path.join(csrc, name), "rb") as f:
                h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()[:16]


def read_traffic_profile(n: int) -> tuple[dict, str | None]:
    """{kernel name: (read MB, write MB)} from the committed counter summary, and the reason it
    cannot be used (None when it can): other N, missing, or measured on other machine code.  A row
    is used only while the kernel in the library being run has the instruction-stream digest the
    summary lists for it (``kfold_amd/kernel_isa.json``, written by the build)."""
    if n != 768:
        return {}, f"the committed counter runs are at N=768, not N={n}"
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return {}, "no counter summary under profiles/"
    try:
        from kfold_amd.build import ISA_JSON

        built = json.loads(ISA_JSON.read_text())
    except (OSError, ValueError):
        return {}, "kfold_amd/kernel_isa.json is missing: the library was not built by kfold_amd.build"
    measured = {}            # table name -> digest the summary was measured on
    for line in text.splitlines():
        cells = [c.strip() for c in line.split("|")]
        if len(cells) >= 5 and cells[1].startswith("kfh::") and cells[2].startswith("`_Z"):
            if built.get(cells[2].strip("`")) == cells[3].strip("`"):
                measured[cells[1]] = cells[3]
    rows = {}
    for line in text.splitlines():
        cells = [c.strip() for c in line.split("|")]
        if len(cells) >= 8 and cells[1] in measured:
            try:
                rows[cells[1]] = (float(cells[5]), float(cells[6]))
            except ValueError:
                pass
    if not rows:
        return {}, "the counter summary under profiles/ was taken on other machine code of every kernel"
    return rows, None


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


def flash_executed_flops(pm, n: int) -> int:
    """MFMA flops the attention kernel issues for this mask (one direction, 4 heads x 32):
    per (row with a valid key, head, query block, key block with a valid key) one 32x32 score
    tile = QK^T (2*32*32*32) + PV (2*32*32*32); a row with no valid key takes one sum of V per
    (head, pair of query blocks): 2*32*32*32 per key block."""
    import torch

    nb = (n + 31) // 32
    m = pm[0].to(torch.bool).cpu()
    mp = torch.zeros(n, nb * 32, dtype=torch.bool)
    mp[:, :n] = m
    active = mp.view(n, nb, 32).any(-1)                  # [row, key block]
    per_row = active.sum(1)                              # key blocks with a valid key
    valid_rows = per_row > 0
    tile = 2 * (2 * 32 * 32 * 32)
    flops = int(per_row[valid_rows].sum()) * nb * 4 * tile
    flops += int((~valid_rows).sum()) * 4 * ((nb + 1) // 2) * nb * (2 * 32 * 32 * 32)
    return flops


def _median_ms(fn, passes: int) -> float:
    ts = []
    for _ in range(passes):
        t0 = time.perf_counter()
        fn()
        ts.append((time.perf_counter() - t0) * 1e3)
    return statistics.median(ts)


def cpu_baseline(n: int) -> dict:
    """The fp32 oracle (a port of the reference's torch path) on the host cores: the whole block
    at N tokens, median of 3 passes on all threads; plus benchmark config 1 (N=64, fp32, all-ones
    mask) on all threads and on one thread, median of 5 passes each."""
    import torch

    from kfold_amd import synthetic
    from oracle import torch_path as O

    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    blk = O.PairSingleBlock(row_chunk=32).eval()
    synthetic.init_weights_(blk, 0)

    def make(nn, frac):
        z, tok, pm = synthetic.pair_inputs(nn, 128, synthetic.n_pad_for(nn, frac), 0)
        s = synthetic.single_inputs(nn, 384, 1)
        return lambda: blk(z.clone(), s.clone(), pm.float(), tok.float())

    with torch.inference_mode():
        torch.set_num_threads(cores)
        run_c1 = make(64, 0.0)
        run_c1()
        c1_all = _median_ms(run_c1, 5)
        run_n = make(n, 0.12)
        n_all = _median_ms(run_n, 3)
        torch.set_num_threads(1)
        run_c1()
        c1_one = _median_ms(run_c1, 5)
        torch.set_num_threads(cores)
    return {
        "value": round(n_all, 1),
        "unit": f"ms per Pairformer block at N={n}",
        "cores": cores,
        "kind": "port",
        "sample": f"the whole block at N={n} (12 % padding), fp32 torch oracle, median of 3 passes, "
                  f"{cores} threads",
        "config1_n64_ms": {"threads": cores, "value": round(c1_all, 2), "one_thread": round(c1_one, 2),
                           "passes": 5},
    }


class Harness:
    """One block's modules, inputs and stage-selective launches for the per-kernel timings."""

    def __init__(self, n: int, pad_frac: float, std: float = 0.02, seed: int = 0, dev=None):
        import torch

        from kfold_amd import _lib, modules, synthetic

        self.torch, self._lib = torch, _lib
        self.L = _lib.lib()
        self.dev = torch.device("cuda:0") if dev is None else dev
        self.n, self.n_pad = n, synthetic.n_pad_for(n, pad_frac)
        self.block = modules.PairSingleBlock().eval()
        synthetic.init_weights_(self.block, seed, std=std)
        self.block.to(self.dev)
        z0, tok, pm = synthetic.pair_inputs(n, 128, self.n_pad, 0)
        s0 = synthetic.single_inputs(n, 384, 1)
        self.z0 = z0.to(torch.bfloat16).to(self.dev)
        self.s0 = s0.to(torch.bfloat16).to(self.dev)
        self.pm, self.tok = pm.to(self.dev), tok.to(self.dev)
        self.m8 = self.pm.contiguous().view(torch.uint8)
        self.stream = torch.cuda.current_stream(self.dev).cuda_stream
        self.out = torch.empty_like(self.z0)
        pb = self.block.pair_block
        with torch.inference_mode():
            pb.tri_mul_out(self.z0, self.pm)
            pb.tri_att_start(self.z0, self.pm)
            self.block(self.z0.clone(), self.s0.clone(), self.pm, self.tok)   # builds every blob
        self.ta_blob = pb.tri_att_start._hip_attention_cache
        self.tm_blob = pb.tri_mul_out._hip_multiplication_cache
        self.ta_ws_bytes = self.L.kfh_triattn_workspace_bytes(n, 128, 4)
        self.tm_ws_bytes = self.L.kfh_trimul_workspace_bytes(n, 128)
        self.ws = torch.empty(max(self.ta_ws_bytes, self.tm_ws_bytes), dtype=torch.uint8, device=self.dev)

    def triattn_stage(self, which: int, ending: int = 0, residual: bool = False) -> None:
        z = self.z0
        self._lib.check(self.L.kfh_triattn_forward_stages(
            z.data_ptr(), self.m8.data_ptr(), self.ta_blob.data_ptr(), z.data_ptr() if residual else None,
            self.out.data_ptr(), self.ws.data_ptr(), self.ta_ws_bytes, 1, self.n, 128, 4, ending, 1e-5,
            self._lib.KFH_BF16, which, self.stream))

    def trimul_stage(self, which: int, direction: int = 0, residual: bool = False) -> None:
        z = self.z0
        self._lib.check(self.L.kfh_trimul_forward_stages(
            z.data_ptr(), self.m8.data_ptr(), self.tm_blob.data_ptr(), z.data_ptr() if residual else None,
            self.out.data_ptr(), self.ws.data_ptr(), self.tm_ws_bytes, 1, self.n, 128, direction, 1e-5,
            self._lib.KFH_BF16, which, self.stream))

    def flash_ms(self, iters: int) -> float:
        self.triattn_stage(self._lib.KFH_STAGE_IN)
        ts = event_time_ms(lambda: self.triattn_stage(self._lib.KFH_STAGE_CORE), iters)
        return sum(ts) / len(ts)


def per_kernel_table(h: Harness, traffic: dict, iters: int = 10) -> dict:
    """Event-timed launches of each hot kernel on the benchmark shape (residual in place, as in the
    block), with the HBM bytes of the committed counter summary where it is current."""
    L = h._lib
    n = h.n
    from kfold_amd import ops
    from kfold_amd.layers.transition import hip_transition

    z = h.z0.clone()
    runs = {}
    h.trimul_stage(L.KFH_STAGE_IN)
    runs["kfh::trimul_in_kernel"] = lambda: h.trimul_stage(L.KFH_STAGE_IN)
    runs["kfh::contract_kernel"] = lambda: h.trimul_stage(L.KFH_STAGE_CORE)
    runs["kfh::trimul_out_kernel"] = lambda: h.trimul_stage(L.KFH_STAGE_OUT, residual=True)
    res = {}
    for name, fn in runs.items():
        res[name] = statistics.median(event_time_ms(fn, iters))
    h.triattn_stage(L.KFH_STAGE_IN)
    runs = {
        "kfh::triattn_proj_kernel": lambda: h.triattn_stage(L.KFH_STAGE_IN),
        "kfh::flash_strip_kernel": lambda: h.triattn_stage(L.KFH_STAGE_CORE),
        "kfh::triattn_out_kernel": lambda: h.triattn_stage(L.KFH_STAGE_OUT, residual=True),
        "kfh::transition_kernel": lambda: hip_transition(h.block.pair_block.transition_z, z, residual=z,
                                                         mask=h.pm, out=z),
        "kfh::pair_bias_kernel": lambda: ops.pair_bias_project(h.z0, h.block._hip_pair_bias_cache, 16),
    }
    for name, fn in runs.items():
        res[name] = statistics.median(event_time_ms(fn, iters))
    flops = {"kfh::contract_kernel": 256 * n**3, "kfh::flash_strip_kernel": 512 * n**3,
             "kfh::transition_kernel": 98304 * 2 * n**2}
    out = {}
    for name, ms in res.items():
        row = {"ms": round(ms, 4)}
        if name in flops:
            row["tflops"] = round(flops[name] / ms / 1e9, 1)
            row["frac_of_2.5PF"] = round(flops[name] / ms / 1e9 / PEAK_BF16_TFLOPS, 4)
        hit = [v for k, v in traffic.items() if k.startswith(name)]
        if hit:
            mb = hit[0][0] + hit[0][1]
            row.update(measured_MB=round(mb, 1), tb_per_s=round(mb / ms / 1e3, 2),
                       frac_of_8TBs=round(mb / ms / 1e3 / (PEAK_HBM_GBS / 1e3), 4))
        else:
            row.update(measured_MB=None, tb_per_s=None, frac_of_8TBs=None)
        out[name.replace("kfh::", "")] = row
    return out


def trunk_c5(blocks: int = 48, n: int = 1024) -> dict:
    """Benchmark config 5: 48-block trunk forward at N=1024, bf16, 15 % padding."""
    import torch

    from kfold_amd import modules, synthetic

    dev = torch.device("cuda:0")
    trunk = modules.PairformerTrunk(blocks).eval()
    synthetic.init_weights_(trunk, 0)
    trunk.to(dev)
    z0, tok, pm = synthetic.pair_inputs(n, 128, synthetic.n_pad_for(n, 0.15), 0)
    s0 = synthetic.single_inputs(n, 384, 1)
    zb, sb = z0.to(torch.bfloat16).to(dev), s0.to(torch.bfloat16).to(dev)
    pm, tok = pm.to(dev), tok.to(dev)
    ts = []
    with torch.inference_mode():
        for it in range(3):
            z, s = zb.clone(), sb.clone()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            trunk(z, s, pm, tok)
            torch.cuda.synchronize()
            ts.append((time.perf_counter() - t0) * 1e3)
    ms = min(ts[1:])
    fl = block_flops(n)["block"] * blocks
    return {"workload": f"pairformer_trunk_{blocks}x_N{n}", "ms": round(ms, 2),
            "ms_per_block": round(ms / blocks, 3), "tflops": round(fl / ms / 1e9, 1),
            "mfma_frac": round(fl / ms / 1e9 / PEAK_BF16_TFLOPS, 4), "runs_ms": [round(t, 2) for t in ts]}


def config_table() -> list[dict]:
    """Every benchmark configuration once on the GPU: time, TFLOP/s, roofline fraction.  (Parity of
    the same configurations is the business of tests/; the CPU times come from
    ``cpu_baseline_configs``.)"""
    import torch

    from kfold_amd import layers, modules, ops, primitives, synthetic
    from kfold_amd.layers.attention_pair_bias import _parameters

    dev = torch.device("cuda:0")
    rows = []
    with torch.inference_mode():
        hip = modules.PairSingleBlock().eval()
        synthetic.init_weights_(hip, 0)
        hip.to(dev)
        z, tok, pm = synthetic.pair_inputs(64, 128, 0, 0)
        s = synthetic.single_inputs(64, 384, 1)
        zd, sd, pmd, tokd = z.to(dev), s.to(dev), pm.to(dev), tok.to(dev)
        ms = statistics.median(event_time_ms(lambda: hip(zd.clone(), sd.clone(), pmd, tokd), 10))
        fl = block_flops(64)["block"]
        rows.append(dict(config="C1", what="block N=64 fp32 io", hip_ms=ms, tflops=fl / ms / 1e9,
                         roof="launch-latency bound (16 kernels)"))
        for cfg, what, n, npad, mk, fl in [
            ("C2", "tri-mul out N=384", 384, 38, lambda: primitives.TriangleMultiplicationOutgoing(128),
             block_flops(384)["trimul"]),
            ("C2", "tri-mul in N=384", 384, 38, lambda: primitives.TriangleMultiplicationIncoming(128),
             block_flops(384)["trimul"]),
            ("C3", "tri-attn start N=512", 512, 64, lambda: primitives.TriangleAttentionStartingNode(128, 4),
             block_flops(512)["triattn"]),
            ("C3", "tri-attn end N=512", 512, 64, lambda: primitives.TriangleAttentionEndingNode(128, 4),
             block_flops(512)["triattn"]),
        ]:
            m = mk().eval()
            synthetic.init_weights_(m, 0)
            m.to(dev)
            z, _, pm = synthetic.pair_inputs(n, 128, npad, 0)
            zd, pmd = z.bfloat16().to(dev), pm.to(dev)
            ms = statistics.median(event_time_ms(lambda: m(zd, pmd), 10))
            rows.append(dict(config=cfg, what=what, hip_ms=ms, tflops=fl / ms / 1e9,
                             roof=f"MFMA {fl / ms / 1e9 / PEAK_BF16_TFLOPS * 100:.1f} %"))
        n = 768
        hip = modules.PairSingleBlock().eval()
        synthetic.init_weights_(hip, 5)
        hip.to(dev)
        z, tok, pm = synthetic.pair_inputs(n, 128, synthetic.n_pad_for(n, 0.12), 6)
        s = synthetic.single_inputs(n, 384, 7)
        zd, sd, tokd = z.bfloat16().to(dev), s.bfloat16().to(dev), tok.to(dev)
        blob_pb = ops.pair_bias_pack(hip.layernorm_z.weight, hip.layernorm_z.bias, hip.linear_pair_bias.weight,
                                     device=dev)
        att = hip.attention
        blob = ops.apb_pack(att.channel_a, att.num_heads, 0, device=dev, **_parameters(att))

        def hip_c4a():
            tiles = ops.pair_bias_project(zd, blob_pb, 16)
            return ops.apb_forward(sd, None, tiles, tokd, blob, 16, 0, True, False)

        ms = statistics.median(event_time_ms(hip_c4a, 10))
        mb = n * n * 128 * 2 / 1e6
        rows.append(dict(config="C4a", what="APB trunk N=768, bias from z", hip_ms=ms, tflops=4.45e9 / ms / 1e9,
                         roof=f"HBM {mb / ms / 1e3 / 8 * 100:.1f} % (z read, {mb:.0f} MB)"))
        m = layers.SelfAttentionPairBias(768, 16, 384, "diffusion_global").eval()
        synthetic.init_weights_(m, 8)
        m.to(dev)
        g = torch.Generator().manual_seed(9)
        ad = torch.randn(1, 5, n, 768, generator=g).bfloat16().to(dev)
        scd = torch.randn(1, 5, n, 384, generator=g).bfloat16().to(dev)
        bd = torch.randn(1, 1, 16, n, n, generator=g).bfloat16().to(dev)
        md = synthetic.token_mask(n, synthetic.n_pad_for(n, 0.12)).reshape(1, 1, n).to(dev)
        ms = statistics.median(event_time_ms(lambda: m(ad, scd, bd, md), 10))
        rows.append(dict(config="C4b", what="APB diffusion N=768 S=5, dense bias in", hip_ms=ms,
                         tflops=3.85e10 / ms / 1e9, roof=f"MFMA {3.85e10 / ms / 1e9 / PEAK_BF16_TFLOPS * 100:.1f} %"))
        rows += shipping_dim_rows(dev, lambda fn: statistics.median(event_time_ms(fn, 10)))
    return rows


def shipping_dim_rows(dev, time_ms, n_wide: int = 768, n_templates: int = 384, n_atoms_windows: int = 24,
                      n_tokens: int = 768) -> list[dict]:
    """The widths the shipping model runs at (configs/kfold.yaml of the reference): triangle
    multiplication and the trunk's TriangularBlock at c_z = 256, triangle attention at c = 64 with
    4 heads of 16 over a batch of 4 templates, and the diffusion attention in fp32 arithmetic.
    ``time_ms(fn)`` returns the time of one call of ``fn`` in ms."""
    import torch

    from kfold_amd import layers, modules, primitives, synthetic

    rows = []
    n = n_wide
    tok = synthetic.token_mask(n, synthetic.n_pad_for(n, 0.12))
    pm = synthetic.pair_mask_from_tokens(tok).to(dev)
    g = torch.Generator().manual_seed(3)
    zd = torch.randn(1, n, n, 256, generator=g).bfloat16().to(dev)
    fl_tm = 2 * n**3 * 256 + n * n * (8 * 256 * 256 + 2 * 256 * 256 + 2 * 256 * 256)      # 2 N^3 D + N^2 (8 C D + 2 D C + 2 C^2) with C = D = 256
    for what, mk in (("tri-mul out C=256", lambda: primitives.TriangleMultiplicationOutgoing(256)),
                     ("tri-mul in C=256", lambda: primitives.TriangleMultiplicationIncoming(256))):
        m = mk().eval()
        synthetic.init_weights_(m, 0)
        m.to(dev)
        ms = time_ms(lambda: m(zd, pm))
        rows.append(dict(config="F2", what=f"{what} N={n}", hip_ms=ms, tflops=fl_tm / ms / 1e9,
                         roof=f"MFMA {fl_tm / ms / 1e9 / PEAK_BF16_TFLOPS * 100:.1f} %"))
    blk = modules.TriangularBlock(256).eval()
    synthetic.init_weights_(blk, 1)
    blk.to(dev)
    fl_blk = 2 * fl_tm + 6 * 256 * 256 * 4 * n * n
    zin = zd.clone()
    ms = time_ms(lambda: blk(zin, pm))
    rows.append(dict(config="F2", what=f"TriangularBlock C=256 N={n} (tri-mul out, in, transition x4)", hip_ms=ms,
                     tflops=fl_blk / ms / 1e9, roof=f"MFMA {fl_blk / ms / 1e9 / PEAK_BF16_TFLOPS * 100:.1f} %"))
    del zd, zin
    n, batch = n_templates, 4
    xd = torch.randn(batch, n, n, 64, generator=g).bfloat16().to(dev)
    pmt = synthetic.pair_mask_from_tokens(synthetic.token_mask(n, synthetic.n_pad_for(n, 0.1))).expand(batch, n, n)
    pmt = pmt.contiguous().to(dev)
    fl_ta = batch * (4 * n**3 * 64 + n * n * (8 * 64 * 64 + 2 * 64 * 4 + 2 * 64 * 64))
    for what, mk in (("tri-attn start", lambda: primitives.TriangleAttentionStartingNode(64, 4)),
                     ("tri-attn end", lambda: primitives.TriangleAttentionEndingNode(64, 4))):
        m = mk().eval()
        synthetic.init_weights_(m, 2)
        m.to(dev)
        ms = time_ms(lambda: m(xd, pmt))
        rows.append(dict(config="F2", what=f"{what} C=64 4x16, {batch} templates, N={n}", hip_ms=ms,
                         tflops=fl_ta / ms / 1e9, roof=f"MFMA {fl_ta / ms / 1e9 / PEAK_BF16_TFLOPS * 100:.1f} %"))
    # diffusion attention on fp32 tensors: fp32 arithmetic (six bf16 part products per k-step)
    n = n_tokens
    m = layers.SelfAttentionPairBias(768, 16, 384, "diffusion_global").eval()
    synthetic.init_weights_(m, 8)
    m.to(dev)
    ad = torch.randn(1, 5, n, 768, generator=g).to(dev)
    scd = torch.randn(1, 5, n, 384, generator=g).to(dev)
    bd = torch.randn(1, 1, 16, n, n, generator=g).to(dev)
    md = synthetic.token_mask(n, synthetic.n_pad_for(n, 0.12)).reshape(1, 1, n).to(dev)
    ms = time_ms(lambda: m(ad, scd, bd, md))
    fl = 3.85e10 * (n / 768) ** 2
    rows.append(dict(config="F3", what=f"APB diffusion N={n} S=5, fp32 arithmetic", hip_ms=ms, tflops=fl / ms / 1e9,
                     roof=f"MFMA {6 * fl / ms / 1e9 / PEAK_BF16_TFLOPS * 100:.1f} % of bf16 peak on the 6x executed products"))
    W = n_atoms_windows
    cross = layers.CrossAttentionPairBias(128, 4, 128).eval()
    synthetic.init_weights_(cross, 9)
    cross.to(dev)
    aq, ak = torch.randn(5, W, 32, 128, generator=g).to(dev), torch.randn(5, W, 128, 128, generator=g).to(dev)
    sq, sk = torch.randn(5, W, 32, 128, generator=g).to(dev), torch.randn(5, W, 128, 128, generator=g).to(dev)
    cb = torch.randn(1, W, 4, 32, 128, generator=g).to(dev)
    cm = torch.ones(1, W, 128, dtype=torch.bool).to(dev)
    ms = time_ms(lambda: cross(aq, ak, sq, sk, cb, cm))
    rows.append(dict(config="F3", what=f"cross attention, 5 x {W} windows of 32 x 128, fp32 arithmetic", hip_ms=ms,
                     tflops=None, roof="launch-latency bound"))
    return rows


def cpu_baseline_configs() -> dict:
    """CPU oracle times of the benchmark configurations (median of 3 passes, all threads); one block
    at N=1024 stands for config 5 (48 such blocks)."""
    import torch

    from kfold_amd import synthetic
    from oracle import torch_path as O

    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
    torch.set_num_threads(cores)
    out = {"threads": cores}

    def timed(fn, passes=3):
        fn()
        return round(_median_ms(fn, passes), 1)

    with torch.inference_mode():
        for key, n, npad, mk in [
            ("C2 tri-mul out N=384", 384, 38, lambda: O.TriangleMultiplicationOutgoing(128)),
            ("C2 tri-mul in N=384", 384, 38, lambda: O.TriangleMultiplicationIncoming(128)),
            ("C3 tri-attn start N=512", 512, 64, lambda: O.TriangleAttentionStartingNode(128, 4, row_chunk=64)),
            ("C3 tri-attn end N=512", 512, 64, lambda: O.TriangleAttentionEndingNode(128, 4, row_chunk=64)),
        ]:
            ref = mk().eval()
            synthetic.init_weights_(ref, 0)
            z, _, pm = synthetic.pair_inputs(n, 128, npad, 0)
            out[key] = timed(lambda: ref(z, pm.float()))
        n = 768
        ref = O.PairSingleBlock().eval()
        synthetic.init_weights_(ref, 5)
        z, tok, _ = synthetic.pair_inputs(n, 128, synthetic.n_pad_for(n, 0.12), 6)
        s = synthetic.single_inputs(n, 384, 7)

        def c4a():
            bias = ref.linear_pair_bias(ref.layernorm_z(z)).movedim(-1, -3)
            return ref.attention(s, None, bias, tok.float())

        out["C4a APB trunk N=768"] = timed(c4a)
        ref2 = O.SelfAttentionPairBias(768, 16, 384, "diffusion_global").eval()
        synthetic.init_weights_(ref2, 8)
        g = torch.Generator().manual_seed(9)
        a = torch.randn(1, 5, n, 768, generator=g)
        sc = torch.randn(1, 5, n, 384, generator=g)
        bias = torch.randn(1, 1, 16, n, n, generator=g)
        mask = synthetic.token_mask(n, synthetic.n_pad_for(n, 0.12)).reshape(1, 1, n)
        out["C4b APB diffusion N=768 S=5"] = timed(lambda: ref2(a, sc, bias, mask))
        blk = O.PairSingleBlock(row_chunk=32).eval()
        synthetic.init_weights_(blk, 0)
        z, tok, pm = synthetic.pair_inputs(1024, 128, synthetic.n_pad_for(1024, 0.15), 0)
        s = synthetic.single_inputs(1024, 384, 1)
        out["C5 one block of 48 at N=1024"] = timed(lambda: blk(z.clone(), s.clone(), pm.float(), tok.float()), 1)
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--n", type=int, default=768, help="tokens (the metric is quoted at 768)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the per-kernel table, the unpadded / large-logit timings and the 48-block trunk")
    ap.add_argument("--table", action="store_true", help="also measure every benchmark configuration")
    ap.add_argument("--phase-chunks", type=int, default=0,
                    help="also time the block with every triangle op's core and output phase overlapped over this "
                         "many ranges of rows (same results bit for bit; reported beside the headline, never as it)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); "
              f"--gpus {args.gpus} is not supported", file=sys.stderr)
        return 2

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no ROCm GPU visible", file=sys.stderr)
        return 1
    from kfold_amd import _lib

    _lib.lib()                                         # fail loudly if the library is not built
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    n = args.n
    h = Harness(n, 0.12)
    block, pm, tok = h.block, h.pm, h.tok
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
        from kfold_amd import modules

        # K steps = K applications of the block, each on the output of the one before, scheduled
        # as a trunk schedules its blocks: the single track of a step runs on a second stream
        # beside the pair track of the next step (bit-identical to the serial order).
        side = torch.cuda.Stream(device=dev)

        def chain(k, z, s, overlap):
            modules.run_blocks([block] * k, z, s, pm, tok, side if overlap else None)

        timings = {}
        for name, overlap in (("serial", False), ("overlapped", True)):
            z, s = h.z0.clone(), h.s0.clone()
            chain(args.warmup, z, s, overlap)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            chain(args.steps, z, s, overlap)
            torch.cuda.synchronize()
            timings[name] = (time.perf_counter() - t0) * 1e3 / args.steps
        ms_per_step = timings["overlapped"]
        if args.phase_chunks > 1:
            block.pair_block.phase_row_chunks = args.phase_chunks
            try:
                for name, overlap in (("phases_serial_tracks", False), ("phases_overlapped_tracks", True)):
                    z, s = h.z0.clone(), h.s0.clone()
                    chain(args.warmup, z, s, overlap)
                    torch.cuda.synchronize()
                    t0 = time.perf_counter()
                    chain(args.steps, z, s, overlap)
                    torch.cuda.synchronize()
                    timings[name] = (time.perf_counter() - t0) * 1e3 / args.steps
            finally:
                block.pair_block.phase_row_chunks = 1

        # ---- per-op times (fresh inputs so the values are those of the first block) ---------
        zb, sb = h.z0, h.s0.clone()
        pb = block.pair_block
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
        flash_avg = h.flash_ms(max(args.steps, 10))
        flash_flops = 512 * n**3                        # QK^T + PV, 4 heads x 32, every tile
        executed = flash_executed_flops(pm, n)
        achieved = flash_flops / flash_avg / 1e9
        traffic, why_not = read_traffic_profile(n)
        fkey = [k for k in traffic if k.startswith("kfh::flash_strip_kernel")]
        traffic_bytes = int(round(sum(traffic[fkey[0]]) * 1e6)) if fkey else None

        extras = {}
        if not args.no_extras:
            extras["kernels"] = per_kernel_table(h, traffic)
            # the same kernel without padding (every tile is executed) ...
            h_full = Harness(n, 0.0)
            full_ms = h_full.flash_ms(10)
            # ... and with weights at std 0.1 (logits a few units wide instead of a few tenths)
            h_wide = Harness(n, 0.12, std=0.1)
            wide_ms = h_wide.flash_ms(10)
            del h_full, h_wide
            extras["flash_variants"] = {
                "no_padding": {"avg_launch_ms": round(full_ms, 4),
                               "tflops": round(flash_flops / full_ms / 1e9, 1),
                               "frac": round(flash_flops / full_ms / 1e9 / PEAK_BF16_TFLOPS, 4)},
                "weights_std_0.1": {"avg_launch_ms": round(wide_ms, 4),
                                    "tflops": round(flash_flops / wide_ms / 1e9, 1)},
            }
            torch.cuda.empty_cache()
            extras["config5_trunk"] = trunk_c5()

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
        "config": {"workload": f"pairformer_block_N{n}", "n_tokens": n, "n_padded_tokens": h.n_pad,
                   "c_z": 128, "c_s": 384, "tri_heads": "4x32", "apb_heads": "16x24",
                   "pair_transition_expansion": 2, "single_transition_expansion": 4,
                   "schedule": "chain of `steps` blocks; single track of step k on a second stream beside the "
                               "pair track of step k+1 (serial_schedule_ms_per_step: everything on one stream)"},
        "schedule": "single track of step k on a second stream beside the pair track of step k+1",
        "serial_schedule_ms_per_step": round(timings["serial"], 4),
        **({"phase_overlap": {"row_chunks": args.phase_chunks,
                              "ms_per_step_tracks_serial": round(timings["phases_serial_tracks"], 4),
                              "ms_per_step_tracks_overlapped": round(timings["phases_overlapped_tracks"], 4)}}
           if "phases_serial_tracks" in timings else {}),
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
            "traffic": traffic_bytes,
            "traffic_note": why_not or "FETCH_SIZE + WRITE_SIZE of profiles/hot_path_kernels_n768_hbm_traffic.txt",
            "avg_launch_ms": round(flash_avg, 4),
            "flops_per_launch": flash_flops,
            "executed_flops": executed,
            "executed_tflops": round(executed / flash_avg / 1e9, 1),
            "executed_frac": round(executed / flash_avg / 1e9 / PEAK_BF16_TFLOPS, 4),
        },
    }
    result.update(extras)
    if args.table:
        rows = config_table()
        result["configs"] = [{k: (round(v, 4) if isinstance(v, float) else v) for k, v in r.items()} for r in rows]
        if not args.no_cpu_baseline:
            result["configs_cpu_ms"] = cpu_baseline_configs()
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(n)
    print(json.dumps(result))
    return 0


def _single_track(block, z, s, tok):
    """The single-track part of the block alone: pair bias from z, attention, transition."""
    from kfold_amd import ops
    from kfold_amd.layers.transition import hip_transition

    tiles = ops.pair_bias_project(z, block._hip_pair_bias_cache, block.num_heads)
    att = block.attention
    ops.apb_forward(s, None, tiles, tok.reshape(1, -1), att._hip_apb_cache, att.num_heads, 0, True, False,
                    residual=s, out=s)
    hip_transition(block.transition, s, residual=s, out=s)


if __name__ == "__main__":
    sys.exit(main())
