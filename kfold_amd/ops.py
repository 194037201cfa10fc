"""Thin functional layer over the C ABI: torch tensors in, torch tensors out.

torch is used for device memory (caching allocator) and the current stream only; every
computation happens inside libkfold_hip.so.  All functions require CUDA (ROCm) tensors.
"""

from __future__ import annotations

import torch

from . import _lib
from ._lib import KFH_BF16, KFH_F32, KFH_INCOMING, KFH_OUTGOING, check

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
        raise NotImplementedError(f"hip triangle multiplication is built for C=128, got {C}")
    ws = _weights_f32(device, ln_in_w, ln_in_b, p_in_w, g_in_w, ln_out_w, ln_out_b, p_out_w, g_out_w)
    blob = torch.empty(nbytes, dtype=torch.uint8, device=device)
    with torch.cuda.device(device):
        check(L.kfh_trimul_pack(*[_ptr(w) for w in ws], KFH_F32, C, blob.data_ptr(), _stream(device)))
    # the fp32 staging copies are released by the caching allocator in stream order
    return blob


def trimul_forward(z: torch.Tensor, mask: torch.Tensor, blob: torch.Tensor, direction: str,
                   eps: float = 1e-5, residual: torch.Tensor | None = None,
                   out: torch.Tensor | None = None) -> torch.Tensor:
    """``out = (residual or 0) + TriangleMultiplication(z, mask)`` for z [*, N, N, C]."""
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
        raise NotImplementedError(f"hip triangle multiplication is built for C=128, got {C}")
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        check(L.kfh_trimul_forward(zc.data_ptr(), m8.data_ptr(), blob.data_ptr(), _ptr(residual),
                                   out.data_ptr(), ws.data_ptr(), ws_bytes, B, N, C,
                                   KFH_INCOMING if direction == "incoming" else KFH_OUTGOING,
                                   float(eps), _io_dtype(zc), _stream(dev)))
    return out


# ---------------------------------------------------------------------------------------
# triangle attention
# ---------------------------------------------------------------------------------------
def triattn_pack(ln_w, ln_b, q_w, k_w, v_w, g_w, bias_w, o_w, device: torch.device) -> torch.Tensor:
    L = _lib.lib()
    C, H = q_w.shape[1], bias_w.shape[0]
    nbytes = L.kfh_triattn_packed_bytes(C, H)
    if nbytes == 0:
        raise NotImplementedError(f"hip triangle attention is built for C=128, H=4; got C={C}, H={H}")
    ws = _weights_f32(device, ln_w, ln_b, q_w, k_w, v_w, g_w, bias_w, o_w)
    blob = torch.empty(nbytes, dtype=torch.uint8, device=device)
    with torch.cuda.device(device):
        check(L.kfh_triattn_pack(*[_ptr(w) for w in ws], KFH_F32, C, H, blob.data_ptr(),
                                 _stream(device)))
    return blob


def triattn_forward(x: torch.Tensor, mask: torch.Tensor | None, blob: torch.Tensor, heads: int,
                    starting: bool, eps: float = 1e-5, residual: torch.Tensor | None = None,
                    out: torch.Tensor | None = None) -> torch.Tensor:
    """``out = (residual or 0) + TriangleAttention(x, mask)`` for x [*, N, N, C]."""
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
            f"hip triangle attention is built for C=128, H=4, N<=8192; got C={C}, H={heads}, N={N}")
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        check(L.kfh_triattn_forward(xc.data_ptr(), m8.data_ptr(), blob.data_ptr(), _ptr(residual),
                                    out.data_ptr(), ws.data_ptr(), ws_bytes, B, N, C, heads,
                                    0 if starting else 1, float(eps), _io_dtype(xc), _stream(dev)))
    return out
