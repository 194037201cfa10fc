"""Host execution model of the HIP kernels — TEST INFRASTRUCTURE, never loaded by the product.

``load()`` builds (if needed) and binds ``libkfold_hostsim.so``: the kernel sources of
``kfold_amd/csrc`` compiled for x86-64 against ``hip/hip_runtime.h`` of this directory, exporting
the C ABI of ``include/kfold_hip.h`` with host pointers.  ``host_backend()`` points the product's
Python layer at that library for the duration of a test, so the modules, the functional layer, the
C ABI and the kernel code itself run on CPU tensors and can be compared with the oracle without a
GPU.  Everything the functional layer allocates inside the context (workspaces, outputs, packed
weights, bias tiles) lies between inaccessible pages and starts out as NaN patterns; the arena the
context yields gives test inputs the same protection.
"""

from __future__ import annotations

import contextlib
import ctypes
import sys
from ctypes import c_int, c_longlong, c_size_t, c_void_p

import torch

import kfold_amd.layers  # noqa: F401  (every module that binds check_inference is imported
import kfold_amd.modules  # noqa: F401   before host_backend() looks for it)
import kfold_amd.primitives  # noqa: F401
from kfold_amd import _lib, ops

from . import build as _build

_sim = None


def load() -> ctypes.CDLL:
    global _sim
    if _sim is None:
        path = _build.build()
        h = ctypes.CDLL(str(path))
        for name, (res, args) in _lib.SIGNATURES.items():
            fn = getattr(h, name)
            fn.restype = res
            fn.argtypes = args
        h.hostsim_alloc.restype = c_void_p
        h.hostsim_alloc.argtypes = [c_size_t, c_size_t]
        h.hostsim_free.restype = None
        h.hostsim_free.argtypes = [c_void_p]
        h.hostsim_set_block_filter.restype = None
        h.hostsim_set_block_filter.argtypes = [c_longlong, c_longlong]
        h.hostsim_set_skip_math.restype = None
        h.hostsim_set_skip_math.argtypes = [c_int]
        h.hostsim_launch_count.restype = c_longlong
        h.hostsim_launch_count.argtypes = []
        h.hostsim_set_schedule.restype = None
        h.hostsim_set_schedule.argtypes = [c_int]
        h.hostsim_set_poison_lds.restype = None
        h.hostsim_set_poison_lds.argtypes = [c_int]
        h.hostsim_set_fill.restype = None
        h.hostsim_set_fill.argtypes = [c_int]
        h.hostsim_report.restype = None
        h.hostsim_report.argtypes = []
        h.hostsim_launch_shapes.restype = c_size_t
        h.hostsim_launch_shapes.argtypes = [ctypes.c_char_p, c_size_t]
        h.hostsim_threads.restype = c_int
        h.hostsim_threads.argtypes = []
        _sim = h
    return _sim


class _Arena:
    """Guard-paged buffers alive until ``release()``."""

    def __init__(self):
        self.ptrs: list[int] = []

    def bytes(self, n: int, align: int = 256) -> torch.Tensor:
        L = load()
        p = L.hostsim_alloc(max(n, 1), align)
        if not p:
            raise MemoryError(f"hostsim_alloc({n})")
        self.ptrs.append(p)
        buf = (ctypes.c_ubyte * max(n, 1)).from_address(p)
        return torch.frombuffer(buf, dtype=torch.uint8)[:n]

    def like(self, t: torch.Tensor, align: int = 16) -> torch.Tensor:
        """A guarded copy of ``t`` (contiguous): the byte after its last element's alignment
        unit is inaccessible."""
        tc = t.detach().contiguous()
        raw = self.bytes(tc.numel() * tc.element_size(), align)
        g = raw.view(tc.dtype).view(tc.shape) if tc.numel() else tc.clone()
        g.copy_(tc)
        return g

    def release(self) -> None:
        L = load()
        for p in self.ptrs:
            L.hostsim_free(p)
        self.ptrs.clear()


class _GuardedTorch:
    """Stands where ``torch`` stands in ``kfold_amd.ops`` while the host backend is active: the
    buffers that module allocates (outputs, packed weights, bias tiles) come from the arena —
    between inaccessible pages, pre-filled with 0xFF — everything else is torch's."""

    def __init__(self, arena: "_Arena"):
        self._arena = arena

    def __getattr__(self, name):
        return getattr(torch, name)

    def empty(self, *size, dtype=torch.float32, device=None):
        shape = tuple(size[0]) if len(size) == 1 and isinstance(size[0], (tuple, list, torch.Size)) else size
        n = 1
        for d in shape:
            n *= int(d)
        esz = torch.empty((), dtype=dtype).element_size()
        raw = self._arena.bytes(n * esz, 16)
        return raw.view(dtype).view(shape) if n else torch.empty(shape, dtype=dtype)

    def empty_like(self, t):
        return self.empty(tuple(t.shape), dtype=t.dtype)


class HostDevice(str):
    """Device name for the twins of GPU tests: ``t.to(HostDevice("cpu"))`` copies, as a transfer to
    a GPU does, so a test that mutates the "device" tensor leaves its host original alone."""


class _NullStream:
    cuda_stream = None


_tensor_to = torch.Tensor.to


def _to_host_copy(self, *args, **kwargs):
    if args and isinstance(args[0], HostDevice):
        return _tensor_to(self, "cpu", *args[1:], **kwargs).clone()
    return _tensor_to(self, *args, **kwargs)


def _cpu_device(*tensors):
    for t in tensors:
        if t is not None:
            return t.device
    return torch.device("cpu")


@contextlib.contextmanager
def host_backend(block_stride: int = 1, block_edge: int = 0, skip_math: bool = False):
    """Route ``kfold_amd`` to the host execution model.  Yields an arena for guarded tensors.

    ``block_stride`` / ``block_edge``: run only every ``block_stride``-th workgroup of each launch
    plus the first and last ``block_edge`` (results are then incomplete: for walking addresses of
    large shapes).  ``skip_math``: MFMAs leave their accumulator unchanged."""
    L = load()
    arena = _Arena()
    saved = {
        "lib": _lib._lib, "require": ops._require_cuda, "stream": ops._stream,
        "workspace": ops._workspace, "device": torch.cuda.device,
        "synchronize": torch.cuda.synchronize, "current_stream": torch.cuda.current_stream,
        "to": torch.Tensor.to, "torch": ops.torch,
    }
    checks = []
    for name, mod in list(sys.modules.items()):
        if name.startswith("kfold_amd") and hasattr(mod, "check_inference"):
            checks.append((mod, mod.check_inference))

    def check_inference(x, what):
        if torch.is_grad_enabled():
            raise RuntimeError(f"The hip {what} backend is inference-only.")

    def workspace(given, need, dev):
        if given is not None:
            return saved["workspace"](given, need, dev)
        return arena.bytes(need)

    _lib._lib = L
    ops._require_cuda = _cpu_device
    ops._stream = lambda dev: None
    ops._workspace = workspace
    ops.torch = _GuardedTorch(arena)
    torch.cuda.device = lambda dev: contextlib.nullcontext()
    torch.cuda.synchronize = lambda *a, **k: None
    torch.cuda.current_stream = lambda *a, **k: _NullStream()
    torch.Tensor.to = _to_host_copy
    for mod, _ in checks:
        mod.check_inference = check_inference
    L.hostsim_set_block_filter(block_stride, block_edge)
    L.hostsim_set_skip_math(1 if skip_math else 0)
    L.hostsim_set_fill(0 if skip_math else 1)      # a walk over addresses needs no NaN pattern
    try:
        yield arena
    finally:
        L.hostsim_set_block_filter(1, 0)
        L.hostsim_set_skip_math(0)
        L.hostsim_set_fill(1)
        _lib._lib = saved["lib"]
        ops._require_cuda = saved["require"]
        ops._stream = saved["stream"]
        ops._workspace = saved["workspace"]
        ops.torch = saved["torch"]
        torch.cuda.device = saved["device"]
        torch.cuda.synchronize = saved["synchronize"]
        torch.cuda.current_stream = saved["current_stream"]
        torch.Tensor.to = saved["to"]
        for mod, fn in checks:
            mod.check_inference = fn
        arena.release()
