"""Shared helpers for the parity tests."""

from __future__ import annotations

import torch

# north-star tolerances of the bf16 HIP path against the fp32 oracle
MAX_ABS = 2e-2
MEAN_ABS = 2e-3
# this repo's own, sharper gate: relative Frobenius error of a bf16 pipeline
REL_FRO = 2e-2


def errors(out: torch.Tensor, ref: torch.Tensor) -> dict:
    o = out.detach().float().cpu()
    r = ref.detach().float().cpu()
    d = (o - r).abs()
    return {
        "max_abs": d.max().item() if d.numel() else 0.0,
        "mean_abs": d.mean().item() if d.numel() else 0.0,
        "rel_fro": ((o - r).norm() / r.norm().clamp_min(1e-30)).item() if d.numel() else 0.0,
        "finite": bool(torch.isfinite(o).all()),
    }


def assert_close(out, ref, what="", max_abs=MAX_ABS, mean_abs=MEAN_ABS, rel_fro=REL_FRO,
                 auto_scale=False):
    """``auto_scale``: for stress cases whose weights are larger than the benchmark's std 0.02
    the outputs are O(1) instead of O(0.1); the absolute tolerances (stated for the benchmark
    scale) then grow with the reference RMS, the relative gate stays as is.  Never used for the
    benchmark configurations themselves."""
    e = errors(out, ref)
    if auto_scale:
        f = max(1.0, ref.detach().float().pow(2).mean().sqrt().item() / 0.2)
        max_abs, mean_abs = max_abs * f, mean_abs * f
    msg = f"{what}: {e}"
    assert e["finite"], msg
    assert e["max_abs"] <= max_abs, msg
    assert e["mean_abs"] <= mean_abs, msg
    if rel_fro is not None:
        assert e["rel_fro"] <= rel_fro, msg
    return e


def ulp_bf16(x: torch.Tensor) -> torch.Tensor:
    """Spacing of bf16 numbers at |x| (8 significant bits)."""
    a = x.detach().float().abs().clamp_min(2.0 ** -126)
    return torch.exp2(torch.floor(torch.log2(a)) - 7)


def assert_stream_close(got, stream_ref, f32_ref, what="", max_flip_frac=2e-4, n_adds=5):
    """A residual stream stored in bf16 (``got``) against the oracle run with the same bf16
    stream rounding (``stream_ref``) and the all-fp32 oracle (``f32_ref``).

    * mean-abs against the bf16-stream oracle: the unscaled north-star limit (2e-3);
    * max-abs: an element of a bf16 stream moves in steps of its spacing (2^-6 for 2 <= |z| < 4,
      2^-5 above), so two correct implementations whose updates differ by far less than the
      limit still land on neighbouring bf16 values now and then ("rounding flips", a random
      walk over the ``n_adds`` in-place adds, one step at most per add).  Elements above the
      unscaled 2e-2 must be rare and within ``n_adds`` bf16 steps of the reference value (plus
      5e-3 for the difference of the updates themselves);
    * control: the distance to the fp32 oracle may not exceed, beyond a small margin, the
      distance of the bf16-stream oracle (exact fp32 arithmetic, same storage) to it — the
      error is then what bf16 storage of the stream costs, not kernel error."""
    g = got.detach().float().cpu()
    s = stream_ref.detach().float().cpu()
    f = f32_ref.detach().float().cpu()
    assert torch.isfinite(g).all(), what
    d = (g - s).abs()
    info = {"mean_abs_vs_stream": d.mean().item(), "max_abs_vs_stream": d.max().item(),
            "frac_above_2e-2": (d > MAX_ABS).float().mean().item(),
            "max_steps_where_above": (d / ulp_bf16(s))[d > MAX_ABS].max().item() if (d > MAX_ABS).any() else 0.0}
    e_hip, e_str = errors(g, f), errors(s, f)
    info.update(hip_vs_f32=e_hip, stream_oracle_vs_f32=e_str)
    msg = f"{what}: {info}"
    assert info["mean_abs_vs_stream"] <= MEAN_ABS, msg
    assert info["frac_above_2e-2"] <= max_flip_frac, msg
    big = d > MAX_ABS
    if big.any():
        assert (d[big] <= n_adds * ulp_bf16(s[big]) + 5e-3).all(), msg
    assert e_hip["max_abs"] <= 1.25 * e_str["max_abs"] + 2e-3, msg
    assert e_hip["mean_abs"] <= 1.1 * e_str["mean_abs"] + 2e-4, msg
    return info
