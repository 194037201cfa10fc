"""fp64 pure-Python/numpy loop restatements of the index formulas of the hot path.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).  These loops are written
from the index form of the reference's torch path, one scalar sum at a time, with no
einsum / matmul / broadcasting, so that a transposed operand, a swapped index, a
dropped term or a wrong chunk half in ``oracle/torch_path.py`` shows up as a
mismatch on tiny sizes (N <= 8).

Weights are passed as dicts of numpy float64 arrays keyed by the reference's
parameter names.
"""

from __future__ import annotations

import math

import numpy as np


def _ln(x, w, b, eps=1e-5):
    """Biased-variance LayerNorm over a 1-D vector (normalization.py:84-90)."""
    n = len(x)
    mu = sum(x) / n
    var = sum((t - mu) ** 2 for t in x) / n
    r = 1.0 / math.sqrt(var + eps)
    return [((x[c] - mu) * r) * (w[c] if w is not None else 1.0) + (b[c] if b is not None else 0.0)
            for c in range(n)]


def _lin(x, W, b=None):
    """y[o] = sum_c W[o][c] x[c] (+ b[o])  (linear.py:97-107; W is [out, in])."""
    return [sum(W[o][c] * x[c] for c in range(len(x))) + (b[o] if b is not None else 0.0)
            for o in range(len(W))]


def _sig(t):
    return 1.0 / (1.0 + math.exp(-t))


def tri_mul(z, mask, p, direction):
    """triangle_multiplication.py:212-229 / :296-313.  z [N,N,C], mask [N,N]."""
    N, _, C = z.shape
    D = C
    xn = [[_ln(z[i, j], p["layernorm_in.weight"], p["layernorm_in.bias"]) for j in range(N)]
          for i in range(N)]
    ab = [[None] * N for _ in range(N)]
    for i in range(N):
        for j in range(N):
            pr = _lin(xn[i][j], p["linear_p_in.weight"])
            gt = _lin(xn[i][j], p["linear_g_in.weight"])
            ab[i][j] = [pr[c] * _sig(gt[c]) * float(mask[i, j]) for c in range(2 * D)]
    out = np.zeros((N, N, C))
    for i in range(N):
        for j in range(N):
            y = [0.0] * D
            for d in range(D):
                acc = 0.0
                for k in range(N):
                    if direction == "outgoing":
                        acc += ab[i][k][d] * ab[j][k][D + d]       # a = first half, b = second
                    else:
                        acc += ab[k][i][d] * ab[k][j][D + d]
                y[d] = acc
            yn = _ln(y, p["layernorm_out.weight"], p["layernorm_out.bias"])
            po = _lin(yn, p["linear_p_out.weight"])
            go = _lin(xn[i][j], p["linear_g_out.weight"])
            for c in range(C):
                out[i, j, c] = po[c] * _sig(go[c])
    return out


def tri_attn(x, mask, p, heads, starting, inf=1e9):
    """triangle_attention.py:375-434 with :246-335.  x [N,N,C], mask [N,N].

    Ending node is written directly in untransposed indices rather than by
    transposing, so that it is an independent check of the transposes.
    """
    N, _, C = x.shape
    dh = C // heads
    xn = [[_ln(x[i, j], p["layer_norm.weight"], p["layer_norm.bias"]) for j in range(N)]
          for i in range(N)]
    q = [[_lin(xn[i][j], p["mha.linear_q.weight"]) for j in range(N)] for i in range(N)]
    k = [[_lin(xn[i][j], p["mha.linear_k.weight"]) for j in range(N)] for i in range(N)]
    v = [[_lin(xn[i][j], p["mha.linear_v.weight"]) for j in range(N)] for i in range(N)]
    g = [[_lin(xn[i][j], p["mha.linear_g.weight"]) for j in range(N)] for i in range(N)]
    tb = [[_lin(xn[i][j], p["linear.weight"]) for j in range(N)] for i in range(N)]  # [i][j][h]
    out = np.zeros((N, N, C))
    for i in range(N):          # the shared index ("row" for starting, "column" for ending)
        for j in range(N):      # the query
            o = [0.0] * C
            for h in range(heads):
                logit = []
                for kk in range(N):
                    if starting:
                        qv, kv, m, b = q[i][j], k[i][kk], mask[i, kk], tb[j][kk][h]
                    else:
                        qv, kv, m, b = q[j][i], k[kk][i], mask[kk, i], tb[kk][j][h]
                    dot = sum(qv[h * dh + c] * kv[h * dh + c] for c in range(dh)) / math.sqrt(dh)
                    logit.append(dot + b - inf * (0.0 if m else 1.0))
                mx = max(logit)
                e = [math.exp(t - mx) for t in logit]
                se = sum(e)
                for c in range(dh):
                    acc = 0.0
                    for kk in range(N):
                        vv = v[i][kk] if starting else v[kk][i]
                        acc += e[kk] / se * vv[h * dh + c]
                    gg = g[i][j] if starting else g[j][i]
                    o[h * dh + c] = acc * _sig(gg[h * dh + c])
            res = _lin(o, p["mha.linear_o.weight"])
            if starting:
                out[i, j] = res
            else:
                out[j, i] = res
    return out


def attention_pair_bias(xq, xk, pair_bias, mask, p, heads, inf=1e9):
    """attention.py:75-94, :239-271.  xq [Lq,C], xk [Lk,C], pair_bias [H,Lq,Lk], mask [Lk]."""
    Lq, C = xq.shape
    Lk = xk.shape[0]
    dh = C // heads
    out = np.zeros((Lq, C))
    kk = [_lin(xk[t], p["linear_k.weight"]) for t in range(Lk)]
    vv = [_lin(xk[t], p["linear_v.weight"]) for t in range(Lk)]
    for qi in range(Lq):
        qq = _lin(xq[qi], p["linear_q.weight"], p.get("linear_q.bias"))
        gg = _lin(xq[qi], p["linear_g.weight"])
        o = [0.0] * C
        for h in range(heads):
            logit = []
            for t in range(Lk):
                dot = sum(qq[h * dh + c] * kk[t][h * dh + c] for c in range(dh)) / math.sqrt(dh)
                logit.append(dot + pair_bias[h, qi, t] - inf * (0.0 if mask[t] else 1.0))
            mx = max(logit)
            e = [math.exp(t - mx) for t in logit]
            se = sum(e)
            for c in range(dh):
                o[h * dh + c] = sum(e[t] / se * vv[t][h * dh + c] for t in range(Lk)) \
                    * _sig(gg[h * dh + c])
        out[qi] = _lin(o, p["linear_out.weight"])
    return out


def transition(x, p):
    """transition.py:48-68 + activation.py:27-29.  x [M, C]."""
    out = np.zeros_like(x)
    for r in range(x.shape[0]):
        xn = _ln(x[r], p["layernorm.weight"], p["layernorm.bias"])
        h = _lin(xn, p["swiglu.linear.weight"])
        half = len(h) // 2
        act = [h[c] * _sig(h[c]) * h[half + c] for c in range(half)]
        out[r] = _lin(act, p["linear_out.weight"])
    return out


def adaln(a, s, p):
    """normalization.py:117-125.  a [M, Ca], s [M, Cs]."""
    out = np.zeros_like(a)
    for r in range(a.shape[0]):
        an = _ln(a[r], None, None)
        sn = _ln(s[r], p["layernorm_s.weight"], None)
        gt = _lin(sn, p["linear_g.weight"], p["linear_g.bias"])
        bs = _lin(sn, p["linear_bias.weight"])
        out[r] = [_sig(gt[c]) * an[c] + bs[c] for c in range(len(an))]
    return out


def parcae_step(z, u, p):
    """model.py:272-277 and :528.  z, u [R, C]; p: layernorm_z.{weight,bias}, parcae_log_a,
    parcae_log_delta [C], parcae_b_cont [C, C] (row = output channel)."""
    R, C = z.shape
    delta = [math.log1p(math.exp(t)) for t in p["parcae_log_delta"]]
    a = [math.exp(-delta[c] * math.exp(p["parcae_log_a"][c])) for c in range(C)]
    out = np.zeros((R, C))
    for r in range(R):
        un = _ln(u[r], p["layernorm_z.weight"], p["layernorm_z.bias"])
        for o in range(C):
            acc = 0.0
            for c in range(C):
                acc += delta[o] * p["parcae_b_cont"][o][c] * un[c]
            out[r, o] = a[o] * z[r, o] + acc
    return out
