"""Thin functional layer over the C ABI: torch tensors in, torch tensors out.

torch is used for device memory (caching allocator) and the current stream only; every
computation happens inside libkfold_hip.so.  All functions require CUDA (ROCm) tensors.
"""

from __future__ import annotations

import torch

from . import _lib
from ._lib import KFH_ARITH_BF16, KFH_ARITH_F32, KFH_BF16, KFH_F32, KFH_INCOMING, KFH_OUTGOING, check

_IO_DTYPES = {torch.bfloat16: KFH_BF16, torch.float32: KFH_F32}


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def _stream(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _io_dtype(t: torch.Tensor) -> int:
    try:
        return _IO_DTYPES[t.dtype]
    except KeyError:
        raise TypeError(f"hip backend supports bfloat16 and float32 tensors, got {t.dtype}") from None


def _require_cuda(*tensors: torch.Tensor | None) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("The hip backend requires tensors on a ROCm GPU.")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} and {t.device}")
    return dev


def _weights_f32(dev: torch.device, *ws: torch.Tensor | None) -> list[torch.Tensor | None]:
    return [None if w is None else w.detach().to(device=dev, dtype=torch.float32).contiguous()
            for w in ws]


def _mask_bytes(mask: torch.Tensor, shape: torch.Size) -> torch.Tensor:
    m = mask
    if m.dtype != torch.bool:
        m = m != 0
    if m.shape != shape:
        m = torch.broadcast_to(m, shape)
    return m.contiguous().view(torch.uint8)


def _workspace(given: torch.Tensor | None, need: int, dev: torch.device) -> torch.Tensor:
    """Scratch memory of a forward call: the caller's buffer if it passed one (reused across calls,
    e.g. one buffer for all ops of a block that run on one stream), else a fresh allocation."""
    if given is None:
        return torch.empty(need, dtype=torch.uint8, device=dev)
    if given.dtype != torch.uint8 or given.device != dev or not given.is_contiguous():
        raise ValueError("workspace must be a contiguous uint8 tensor on the device of the inputs")
    if given.numel() < need:
        raise ValueError(f"workspace holds {given.numel()} bytes, this call needs {need}")
    if given.data_ptr() % 256:
        raise ValueError("workspace must be aligned to 256 bytes")
    return given


# a batch is taken through the kernels at once when its workspace stays below this many bytes
_BATCHED_WORKSPACE_CAP = 32 << 30


def _batched_need(per_element: int, batched: int, given: torch.Tensor | None) -> int:
    """Workspace size to ask for: the batched size if it is affordable (or the caller's buffer
    already holds it), else the per-element size (batch elements then run in turn)."""
    if batched > per_element and (batched <= _BATCHED_WORKSPACE_CAP if given is None else given.numel() >= batched):
        return batched
    return per_element


def row_ranges(n: int, chunks: int, granule: int) -> list[tuple[int, int]]:
    """[0, n) cut into at most ``chunks`` ranges (row0, nrows) that start at multiples of ``granule``
    and are as even as the granule allows."""
    blocks = (n + granule - 1) // granule
    k = max(1, min(chunks, blocks))
    out, b0 = [], 0
    for c in range(k):
        b1 = b0 + (blocks - b0) // (k - c)
        r0, r1 = b0 * granule, min(b1 * granule, n)
        out.append((r0, r1 - r0))
        b0 = b1
    return out


def _run_phased(call, n: int, ranges, dev: torch.device, side, before_write=None) -> None:
    """One op in phases over row ranges.  ``call(stages, row0, nrows)`` enqueues on the current
    stream.  The input phase covers all rows; then the core phase of range c+1 (compute-bound) is
    enqueued on the caller's stream while the output phase of range c (memory-bound) runs on ``side``.
    Without ``side`` everything runs in order on the caller's stream.  Either way the kernels are those
    of the whole op on offset pointers: same bits."""
    call(_lib.KFH_STAGE_IN, 0, n)
    if before_write is not None:
        before_write()                         # the first output phase below writes
    if side is None:
        for r0, nr in ranges:
            call(_lib.KFH_STAGE_CORE, r0, nr)
            call(_lib.KFH_STAGE_OUT, r0, nr)
        return
    main = torch.cuda.current_stream(dev)
    for r0, nr in ranges:
        call(_lib.KFH_STAGE_CORE, r0, nr)
        done = torch.cuda.Event()
        done.record(main)
        with torch.cuda.stream(side):
            side.wait_event(done)
            call(_lib.KFH_STAGE_OUT, r0, nr)
    main.wait_stream(side)


def workspace_bytes(op: str, **shape) -> int:
    """Bytes of scratch memory a forward call needs (0: shape not supported): ``trimul`` (N, C),
    ``triattn`` (N, C, heads) — both also with ``B``: the size that takes a batch through the kernels at
    once —, ``transition`` (rows, C, expansion), ``apb`` (S, L, C, heads,
    cond_channels, arith), ``cross_apb`` (W, Lq, Lk, C, heads, cond_channels, arith).  Needs no GPU."""
    L = _lib.lib()
    g = shape.__getitem__
    if op == "trimul":
        if "B" in shape:
            return L.kfh_trimul_workspace_bytes_batched(g("B"), g("N"), g("C"))
        return L.kfh_trimul_workspace_bytes(g("N"), g("C"))
    if op == "triattn":
        if "B" in shape:
            return L.kfh_triattn_workspace_bytes_batched(g("B"), g("N"), g("C"), g("heads"))
        return L.kfh_triattn_workspace_bytes(g("N"), g("C"), g("heads"))
    if op == "transition":
        return L.kfh_transition_workspace_bytes(g("rows"), g("C"), g("expansion"))
    if op == "apb":
        return L.kfh_apb_workspace_bytes(g("S"), g("L"), g("C"), g("heads"), shape.get("cond_channels", 0),
                                         shape.get("arith", KFH_ARITH_BF16))
    if op == "cross_apb":
        return L.kfh_cross_apb_workspace_bytes(g("W"), g("Lq"), g("Lk"), g("C"), g("heads"),
                                               shape.get("cond_channels", 0), shape.get("arith", KFH_ARITH_BF16))
    raise ValueError(f"unknown op {op!r}")


# ---------------------------------------------------------------------------------------
# triangle multiplication
# ---------------------------------------------------------------------------------------
def trimul_pack(ln_in_w, ln_in_b, p_in_w, g_in_w, ln_out_w, ln_out_b, p_out_w, g_out_w,
                device: torch.device) -> torch.Tensor:
    """Pack one module's weights into the kernel's fragment-order blob (uint8 tensor)."""
    L = _lib.lib()
    C = p_out_w.shape[0]
    nbytes = L.kfh_trimul_packed_bytes(C)
    if nbytes == 0:
        raise NotImplementedError(f"hip triangle multiplication takes C a multiple of 32 up to 256, got {C}")
    ws = _weights_f32(device, ln_in_w, ln_in_b, p_in_w, g_in_w, ln_out_w, ln_out_b, p_out_w, g_out_w)
    blob = torch.empty(nbytes, dtype=torch.uint8, device=device)
    with torch.cuda.device(device):
        check(L.kfh_trimul_pack(*[_ptr(w) for w in ws], KFH_F32, C, blob.data_ptr(), _stream(device)))
    # the fp32 staging copies are released by the caching allocator in stream order
    return blob


def trimul_forward(z: torch.Tensor, mask: torch.Tensor, blob: torch.Tensor, direction: str,
                   eps: float = 1e-5, residual: torch.Tensor | None = None,
                   out: torch.Tensor | None = None, before_write=None,
                   workspace: torch.Tensor | None = None, row_chunks: int = 1,
                   side: "torch.cuda.Stream | None" = None) -> torch.Tensor:
    """``out = (residual or 0) + TriangleMultiplication(z, mask)`` for z [*, N, N, C].

    ``row_chunks`` > 1 (one batch element, C = 128 or 256): contraction and output phase run over
    that many ranges of result rows, the output phase of a range on the stream ``side`` (if given)
    beside the contraction of the next range; results are the same bits as with one range.

    ``workspace``: optional uint8 scratch tensor of at least ``workspace_bytes("trimul", N=, C=)``
    bytes to use instead of allocating one (its contents are overwritten).

    ``before_write``: called after the kernels that only read ``z`` have been enqueued and before
    the one that writes ``out`` (which may be ``z``): the place to make this stream wait for
    another stream's reads of ``z``."""
    dev = _require_cuda(z, mask, blob, residual, out)
    if direction not in ("outgoing", "incoming"):
        raise ValueError(f"unknown direction: {direction!r} (expected 'outgoing'/'incoming')")
    N, C = z.shape[-2], z.shape[-1]
    if z.dim() < 3 or z.shape[-3] != N:
        raise ValueError(f"expected z of shape [*, N, N, C], got {tuple(z.shape)}")
    B = z.numel() // (N * N * C) if z.numel() else 0
    zc = z.contiguous()
    m8 = _mask_bytes(mask, z.shape[:-1])
    if out is None:
        out = torch.empty_like(zc)
    elif out.shape != z.shape or out.dtype != z.dtype or not out.is_contiguous():
        raise ValueError("out must be contiguous with the shape and dtype of z")
    if residual is not None and (residual.shape != z.shape or residual.dtype != z.dtype
                                 or not residual.is_contiguous()):
        raise ValueError("residual must be contiguous with the shape and dtype of z")
    if B == 0:
        return out
    L = _lib.lib()
    ws_bytes = L.kfh_trimul_workspace_bytes(N, C)
    if ws_bytes == 0:
        raise NotImplementedError(f"hip triangle multiplication takes C a multiple of 32 up to 256, got {C}")
    if B > 1:
        ws_bytes = _batched_need(ws_bytes, L.kfh_trimul_workspace_bytes_batched(B, N, C), workspace)
    ws = _workspace(workspace, ws_bytes, dev)
    d = KFH_INCOMING if direction == "incoming" else KFH_OUTGOING
    granule = L.kfh_trimul_row_granule(N, C) if row_chunks > 1 and B == 1 else 0
    ranges = row_ranges(N, row_chunks, granule) if granule else []
    with torch.cuda.device(dev):
        if len(ranges) > 1:
            head = (zc.data_ptr(), m8.data_ptr(), blob.data_ptr(), _ptr(residual), out.data_ptr(),
                    ws.data_ptr(), ws_bytes, B, N, C, d, float(eps), _io_dtype(zc))
            _run_phased(lambda st, r0, nr: check(L.kfh_trimul_forward_rows(*head, st, r0, nr, _stream(dev))),
                        N, ranges, dev, side, before_write)
        elif before_write is None or B != 1:
            if before_write is not None:
                before_write()
            check(L.kfh_trimul_forward(zc.data_ptr(), m8.data_ptr(), blob.data_ptr(), _ptr(residual),
                                       out.data_ptr(), ws.data_ptr(), ws_bytes, B, N, C, d,
                                       float(eps), _io_dtype(zc), _stream(dev)))
        else:
            args = (zc.data_ptr(), m8.data_ptr(), blob.data_ptr(), _ptr(residual), out.data_ptr(),
                    ws.data_ptr(), ws_bytes, B, N, C, d, float(eps), _io_dtype(zc))
            check(L.kfh_trimul_forward_stages(*args, _lib.KFH_STAGE_IN | _lib.KFH_STAGE_CORE, _stream(dev)))
            before_write()
            check(L.kfh_trimul_forward_stages(*args, _lib.KFH_STAGE_OUT, _stream(dev)))
    return out


# ---------------------------------------------------------------------------------------
# triangle attention
# ---------------------------------------------------------------------------------------
def triattn_pack(ln_w, ln_b, q_w, k_w, v_w, g_w, bias_w, o_w, device: torch.device) -> torch.Tensor:
    L = _lib.lib()
    C, H = q_w.shape[1], bias_w.shape[0]
    nbytes = L.kfh_triattn_packed_bytes(C, H)
    if nbytes == 0:
        raise NotImplementedError(f"hip triangle attention takes C a multiple of 32 and head dim <= 64; got C={C}, H={H}")
    ws = _weights_f32(device, ln_w, ln_b, q_w, k_w, v_w, g_w, bias_w, o_w)
    blob = torch.empty(nbytes, dtype=torch.uint8, device=device)
    with torch.cuda.device(device):
        check(L.kfh_triattn_pack(*[_ptr(w) for w in ws], KFH_F32, C, H, blob.data_ptr(),
                                 _stream(device)))
    return blob


def triattn_forward(x: torch.Tensor, mask: torch.Tensor | None, blob: torch.Tensor, heads: int,
                    starting: bool, eps: float = 1e-5, residual: torch.Tensor | None = None,
                    out: torch.Tensor | None = None, workspace: torch.Tensor | None = None,
                    row_chunks: int = 1, side: "torch.cuda.Stream | None" = None) -> torch.Tensor:
    """``out = (residual or 0) + TriangleAttention(x, mask)`` for x [*, N, N, C]; ``workspace`` as in
    ``trimul_forward`` (``workspace_bytes("triattn", N=, C=, heads=)``); ``row_chunks`` / ``side`` as in
    ``trimul_forward`` (one batch element, C = 128 with 4 heads; ranges of 64 attention rows at least)."""
    dev = _require_cuda(x, mask, blob, residual, out)
    N, C = x.shape[-2], x.shape[-1]
    if x.dim() < 3 or x.shape[-3] != N:
        raise ValueError(f"expected x of shape [*, N, N, C], got {tuple(x.shape)}")
    B = x.numel() // (N * N * C) if x.numel() else 0
    xc = x.contiguous()
    if mask is None:
        m8 = torch.ones(x.shape[:-1], dtype=torch.uint8, device=dev)
    else:
        m8 = _mask_bytes(mask, x.shape[:-1])
    if out is None:
        out = torch.empty_like(xc)
    elif out.shape != x.shape or out.dtype != x.dtype or not out.is_contiguous():
        raise ValueError("out must be contiguous with the shape and dtype of x")
    if residual is not None and (residual.shape != x.shape or residual.dtype != x.dtype
                                 or not residual.is_contiguous()):
        raise ValueError("residual must be contiguous with the shape and dtype of x")
    if B == 0:
        return out
    L = _lib.lib()
    ws_bytes = L.kfh_triattn_workspace_bytes(N, C, heads)
    if ws_bytes == 0:
        raise NotImplementedError(
            f"hip triangle attention takes C a multiple of 32, head dim <= 64, N <= 8192; got C={C}, H={heads}, N={N}")
    if B > 1:
        ws_bytes = _batched_need(ws_bytes, L.kfh_triattn_workspace_bytes_batched(B, N, C, heads), workspace)
    ws = _workspace(workspace, ws_bytes, dev)
    ranges = row_ranges(N, row_chunks, 64) if row_chunks > 1 and B == 1 and C == 128 and heads == 4 else []
    if ranges and ranges[-1][1] < 48 and len(ranges) > 1:      # fold a short tail into the range before
        (r0, nr), (_, tail) = ranges[-2], ranges[-1]
        ranges[-2:] = [(r0, nr + tail)]
    with torch.cuda.device(dev):
        if len(ranges) > 1:
            head = (xc.data_ptr(), m8.data_ptr(), blob.data_ptr(), _ptr(residual), out.data_ptr(),
                    ws.data_ptr(), ws_bytes, B, N, C, heads, 0 if starting else 1, float(eps), _io_dtype(xc))
            _run_phased(lambda st, r0, nr: check(L.kfh_triattn_forward_rows(*head, st, r0, nr, _stream(dev))),
                        N, ranges, dev, side)
        else:
            check(L.kfh_triattn_forward(xc.data_ptr(), m8.data_ptr(), blob.data_ptr(), _ptr(residual),
                                        out.data_ptr(), ws.data_ptr(), ws_bytes, B, N, C, heads,
                                        0 if starting else 1, float(eps), _io_dtype(xc), _stream(dev)))
    return out


# ---------------------------------------------------------------------------------------
# transition
# ---------------------------------------------------------------------------------------
def transition_pack(ln_w, ln_b, swiglu_w, out_w, device: torch.device) -> torch.Tensor:
    L = _lib.lib()
    C = out_w.shape[0]
    E = out_w.shape[1] // C
    nbytes = L.kfh_transition_packed_bytes(C, E)
    if nbytes == 0:
        raise NotImplementedError(f"hip transition does not support C={C}, expansion={E}")
    ws = _weights_f32(device, ln_w, ln_b, swiglu_w, out_w)
    blob = torch.empty(nbytes, dtype=torch.uint8, device=device)
    with torch.cuda.device(device):
        check(L.kfh_transition_pack(*[_ptr(w) for w in ws], KFH_F32, C, E, blob.data_ptr(),
                                    _stream(device)))
    return blob


def transition_forward(x: torch.Tensor, blob: torch.Tensor, expansion: int, eps: float = 1e-5,
                       residual: torch.Tensor | None = None, mask: torch.Tensor | None = None,
                       out: torch.Tensor | None = None, workspace: torch.Tensor | None = None) -> torch.Tensor:
    """``out = ((residual or 0) + Transition(x)) * (mask or 1)`` over the last dim of x; ``workspace``
    as in ``trimul_forward`` (``workspace_bytes("transition", rows=, C=, expansion=)``)."""
    dev = _require_cuda(x, blob, residual, mask, out)
    C = x.shape[-1]
    rows = x.numel() // C if x.numel() else 0
    xc = x.contiguous()
    if out is None:
        out = torch.empty_like(xc)
    elif out.shape != x.shape or out.dtype != x.dtype or not out.is_contiguous():
        raise ValueError("out must be contiguous with the shape and dtype of x")
    if residual is not None and (residual.shape != x.shape or residual.dtype != x.dtype
                                 or not residual.is_contiguous()):
        raise ValueError("residual must be contiguous with the shape and dtype of x")
    m8 = None if mask is None else _mask_bytes(mask, x.shape[:-1])
    if rows == 0:
        return out
    L = _lib.lib()
    ws_bytes = L.kfh_transition_workspace_bytes(rows, C, expansion)
    ws = _workspace(workspace, ws_bytes, dev) if ws_bytes else None
    with torch.cuda.device(dev):
        check(L.kfh_transition_forward(xc.data_ptr(), blob.data_ptr(), _ptr(residual), _ptr(m8),
                                       out.data_ptr(), _ptr(ws), ws_bytes, rows, C, expansion,
                                       float(eps), _io_dtype(xc), _stream(dev)))
    return out


# ---------------------------------------------------------------------------------------
# pair bias tiles and pair-bias attention
# ---------------------------------------------------------------------------------------
def bias_tiles_from_dense(pair_bias: torch.Tensor, arith: int = KFH_ARITH_BF16) -> torch.Tensor:
    """Dense pair bias [nbatch, H, L, L] -> the attention kernel's bias tiles (flat uint8): bf16
    tiles, or fp32 tiles for ``arith=KFH_ARITH_F32``."""
    dev = _require_cuda(pair_bias)
    nbatch, H, Lq, Lk = pair_bias.shape
    if Lq != Lk:
        raise NotImplementedError("hip pair-bias attention is built for self attention (Lq == Lk)")
    pb = pair_bias.contiguous()
    if pb.dtype not in _IO_DTYPES:
        pb = pb.float()
    L = _lib.lib()
    tiles = torch.empty(L.kfh_bias_tiles_bytes(nbatch, H, Lq, arith), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        check(L.kfh_bias_tiles_from_dense(pb.data_ptr(), _io_dtype(pb), tiles.data_ptr(), nbatch, H, Lq,
                                          arith, _stream(dev)))
    return tiles


def pair_bias_pack(ln_w, ln_b, w, device: torch.device) -> torch.Tensor:
    L = _lib.lib()
    H, C = w.shape
    nbytes = L.kfh_pair_bias_packed_bytes(C, H)
    if nbytes == 0:
        raise NotImplementedError(f"hip pair-bias projection is built for C=128, H<=32; got C={C}, H={H}")
    ws = _weights_f32(device, ln_w, ln_b, w)
    blob = torch.empty(nbytes, dtype=torch.uint8, device=device)
    with torch.cuda.device(device):
        check(L.kfh_pair_bias_pack(*[_ptr(t) for t in ws], KFH_F32, C, H, blob.data_ptr(), _stream(device)))
    return blob


def pair_bias_project(z: torch.Tensor, blob: torch.Tensor, heads: int, eps: float = 1e-5) -> torch.Tensor:
    """tiles of ``linear_pair_bias(LN(z))`` for z [B, N, N, C]; returns the flat tile buffer."""
    dev = _require_cuda(z, blob)
    B, N, N2, C = z.shape
    assert N == N2
    zc = z.contiguous()
    L = _lib.lib()
    tiles = torch.empty(L.kfh_bias_tiles_bytes(B, heads, N, KFH_ARITH_BF16), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        check(L.kfh_pair_bias_project(zc.data_ptr(), blob.data_ptr(), tiles.data_ptr(), B, N, C, heads,
                                      float(eps), _io_dtype(zc), _stream(dev)))
    return tiles


def apb_pack(C: int, H: int, Cs: int, *, ln_w=None, ln_b=None, q_w, q_b, k_w, v_w, g_w, o_w,
             adaln_s_w=None, adaln_g_w=None, adaln_g_b=None, adaln_bias_w=None, ada_out_w=None,
             ada_out_b=None, device: torch.device, arith: int = KFH_ARITH_BF16) -> torch.Tensor:
    L = _lib.lib()
    nbytes = L.kfh_apb_packed_bytes(C, H, Cs, arith)
    if nbytes == 0:
        raise NotImplementedError(
            f"hip pair-bias attention: C={C}, H={H}, Cs={Cs} unsupported "
            "(channels multiples of 128 up to 2048, head dim <= 64)")
    ws = _weights_f32(device, ln_w, ln_b, q_w, q_b, k_w, v_w, g_w, o_w, adaln_s_w, adaln_g_w,
                      adaln_g_b, adaln_bias_w, ada_out_w, ada_out_b)
    blob = torch.empty(nbytes, dtype=torch.uint8, device=device)
    with torch.cuda.device(device):
        check(L.kfh_apb_pack(*[_ptr(t) for t in ws], KFH_F32, C, H, Cs, arith, blob.data_ptr(), _stream(device)))
    return blob


def apb_forward(a: torch.Tensor, s_cond: torch.Tensor | None, tiles: torch.Tensor, mask: torch.Tensor,
                blob: torch.Tensor, heads: int, cond_channels: int, apply_norm: bool,
                bias_per_sample: bool, eps: float = 1e-5, residual: torch.Tensor | None = None,
                out: torch.Tensor | None = None, workspace: torch.Tensor | None = None,
                arith: int = KFH_ARITH_BF16) -> torch.Tensor:
    """a [S, L, C]; s_cond [S or 1, L, Cs] or None; mask [S or 1, L]; tiles from the calls above;
    ``workspace`` as in ``trimul_forward`` (``workspace_bytes("apb", S=, L=, C=, heads=, cond_channels=,
    arith=)``).  ``arith``: the arithmetic the blob and the tiles were made for."""
    dev = _require_cuda(a, s_cond, tiles, mask, blob, residual, out)
    S, Lq, C = a.shape
    ac = a.contiguous()
    m8 = _mask_bytes(mask, mask.shape)
    if m8.shape not in ((S, Lq), (1, Lq)):
        raise ValueError(f"mask shape {tuple(mask.shape)} does not match a {tuple(a.shape)}")
    sc = None
    if s_cond is not None:
        sc = s_cond.contiguous()
        if sc.dtype != ac.dtype:
            sc = sc.to(ac.dtype)
        if sc.shape[0] not in (1, S) or sc.shape[1] != Lq or sc.shape[2] != cond_channels:
            raise ValueError(f"s shape {tuple(s_cond.shape)} does not match a {tuple(a.shape)}")
    if out is None:
        out = torch.empty_like(ac)
    elif out.shape != a.shape or out.dtype != a.dtype or not out.is_contiguous():
        raise ValueError("out must be contiguous with the shape and dtype of a")
    if residual is not None and (residual.shape != a.shape or residual.dtype != a.dtype
                                 or not residual.is_contiguous()):
        raise ValueError("residual must be contiguous with the shape and dtype of a")
    L = _lib.lib()
    ws_bytes = L.kfh_apb_workspace_bytes(S, Lq, C, heads, cond_channels, arith)
    if ws_bytes == 0:
        raise NotImplementedError(f"hip pair-bias attention: unsupported shape S={S} L={Lq} C={C} H={heads}")
    ws = _workspace(workspace, ws_bytes, dev)
    with torch.cuda.device(dev):
        check(L.kfh_apb_forward(ac.data_ptr(), _ptr(sc), tiles.data_ptr(), m8.data_ptr(), blob.data_ptr(),
                                _ptr(residual), out.data_ptr(), ws.data_ptr(), ws_bytes, S, Lq, C, heads,
                                cond_channels, 1 if apply_norm else 0, 1 if bias_per_sample else 0,
                                1 if m8.shape[0] == S and S > 1 else 0,
                                1 if sc is not None and sc.shape[0] == S and S > 1 else 0,
                                float(eps), _io_dtype(ac), arith, _stream(dev)))
    return out


# ---------------------------------------------------------------------------------------
# Parcae recurrence step
# ---------------------------------------------------------------------------------------
def parcae_pack(ln_w, ln_b, log_a, log_delta, b_cont, device: torch.device) -> torch.Tensor:
    L = _lib.lib()
    C = b_cont.shape[0]
    nbytes = L.kfh_parcae_packed_bytes(C)
    if nbytes == 0:
        raise NotImplementedError(f"hip Parcae step is built for C=128 and C=256, got {C}")
    ws = _weights_f32(device, ln_w, ln_b, log_a, log_delta, b_cont)
    blob = torch.empty(nbytes, dtype=torch.uint8, device=device)
    with torch.cuda.device(device):
        check(L.kfh_parcae_pack(*[_ptr(w) for w in ws], KFH_F32, C, blob.data_ptr(), _stream(device)))
    return blob


def parcae_step(z: torch.Tensor, u: torch.Tensor, blob: torch.Tensor, eps: float = 1e-5,
                out: torch.Tensor | None = None, u_add: torch.Tensor | None = None) -> torch.Tensor:
    """``out = a * z + b LN(u [+ u_add])`` over the last dim; ``out`` may be ``z`` (in place)."""
    dev = _require_cuda(z, u, blob, out, u_add)
    if u.shape != z.shape or u.dtype != z.dtype:
        raise ValueError("z and u must have the same shape and dtype")
    if u_add is not None and (u_add.shape != z.shape or u_add.dtype != z.dtype or not u_add.is_contiguous()):
        raise ValueError("u_add must be contiguous with the shape and dtype of z")
    C = z.shape[-1]
    rows = z.numel() // C if z.numel() else 0
    if not z.is_contiguous() or not u.is_contiguous():
        raise ValueError("z and u must be contiguous")
    if out is None:
        out = torch.empty_like(z)
    elif out.shape != z.shape or out.dtype != z.dtype or not out.is_contiguous():
        raise ValueError("out must be contiguous with the shape and dtype of z")
    if rows == 0:
        return out
    L = _lib.lib()
    with torch.cuda.device(dev):
        check(L.kfh_parcae_step(z.data_ptr(), u.data_ptr(), _ptr(u_add), blob.data_ptr(), out.data_ptr(), rows, C,
                                float(eps), _io_dtype(z), _stream(dev)))
    return out


# ---------------------------------------------------------------------------------------
# cross attention with pair bias over local windows
# ---------------------------------------------------------------------------------------
_CROSS_ORDER = ("lnq_w", "lnq_b", "lnk_w", "lnk_b", "q_w", "q_b", "k_w", "v_w", "g_w", "o_w", "adaq_s_w",
                "adaq_g_w", "adaq_g_b", "adaq_bias_w", "adak_s_w", "adak_g_w", "adak_g_b", "adak_bias_w",
                "ada_out_w", "ada_out_b")


def cross_apb_pack(C: int, H: int, Cs: int, device: torch.device, arith: int = KFH_ARITH_BF16,
                   **weights) -> torch.Tensor:
    L = _lib.lib()
    nbytes = L.kfh_cross_apb_packed_bytes(C, H, Cs, arith)
    if nbytes == 0:
        raise NotImplementedError(f"hip cross attention: C={C}, H={H}, Cs={Cs} unsupported")
    ws = _weights_f32(device, *[weights.get(k) for k in _CROSS_ORDER])
    blob = torch.empty(nbytes, dtype=torch.uint8, device=device)
    with torch.cuda.device(device):
        check(L.kfh_cross_apb_pack(*[_ptr(t) for t in ws], KFH_F32, C, H, Cs, arith, blob.data_ptr(),
                                   _stream(device)))
    return blob


def cross_apb_forward(a_q: torch.Tensor, a_k: torch.Tensor, s_q, s_k, pair_bias: torch.Tensor, mask: torch.Tensor,
                      blob: torch.Tensor, heads: int, cond_channels: int, eps: float = 1e-5,
                      residual: torch.Tensor | None = None, out: torch.Tensor | None = None,
                      workspace: torch.Tensor | None = None, apply_norm: bool = True,
                      arith: int = KFH_ARITH_BF16) -> torch.Tensor:
    """a_q [W, Lq, C], a_k [W, Lk, C], s_q / s_k [W, L., Cs] or None, pair_bias [W, H, Lq, Lk], mask [W, Lk];
    ``workspace`` as in ``trimul_forward`` (``workspace_bytes("cross_apb", W=, Lq=, Lk=, C=, heads=,
    cond_channels=, arith=)``).  ``apply_norm=False``: a_q / a_k are already normalised (the functional
    entry); then no conditioning is applied either."""
    dev = _require_cuda(a_q, a_k, s_q, s_k, pair_bias, mask, blob, residual, out)
    W, Lq, C = a_q.shape
    Lk = a_k.shape[1]
    if a_k.shape != (W, Lk, C) or pair_bias.shape != (W, heads, Lq, Lk) or mask.shape != (W, Lk):
        raise ValueError("cross attention: inconsistent window shapes")
    aq, ak = a_q.contiguous(), a_k.contiguous().to(a_q.dtype)
    pb = pair_bias.contiguous()
    if pb.dtype not in _IO_DTYPES:
        pb = pb.float()
    m8 = _mask_bytes(mask, mask.shape)
    sq = sk = None
    if cond_channels and apply_norm:
        sq, sk = s_q.contiguous().to(aq.dtype), s_k.contiguous().to(aq.dtype)
        if sq.shape != (W, Lq, cond_channels) or sk.shape != (W, Lk, cond_channels):
            raise ValueError("cross attention: conditioning shapes do not match")
    if out is None:
        out = torch.empty_like(aq)
    elif out.shape != a_q.shape or out.dtype != a_q.dtype or not out.is_contiguous():
        raise ValueError("out must be contiguous with the shape and dtype of a_q")
    if residual is not None and (residual.shape != a_q.shape or residual.dtype != a_q.dtype
                                 or not residual.is_contiguous()):
        raise ValueError("residual must be contiguous with the shape and dtype of a_q")
    L = _lib.lib()
    ws_bytes = L.kfh_cross_apb_workspace_bytes(W, Lq, Lk, C, heads, cond_channels, arith)
    if ws_bytes == 0:
        raise NotImplementedError(f"hip cross attention: unsupported shape W={W} Lq={Lq} Lk={Lk} C={C} H={heads}")
    ws = _workspace(workspace, ws_bytes, dev)
    with torch.cuda.device(dev):
        check(L.kfh_cross_apb_forward(aq.data_ptr(), ak.data_ptr(), _ptr(sq), _ptr(sk), pb.data_ptr(),
                                      _io_dtype(pb), m8.data_ptr(), blob.data_ptr(), _ptr(residual),
                                      out.data_ptr(), ws.data_ptr(), ws_bytes, W, Lq, Lk, C, heads,
                                      cond_channels, 1 if apply_norm else 0, float(eps), _io_dtype(aq), arith,
                                      _stream(dev)))
    return out
