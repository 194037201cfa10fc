"""ctypes binding of libkfold_hip.so (the C ABI declared in include/kfold_hip.h).

The library is loaded on first use.  There is no fallback: if it has not been built
(``python -m kfold_amd.build``) every entry point raises ``ImportError``.
"""

from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_longlong, c_size_t, c_void_p
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libkfold_hip.so"

KFH_BF16, KFH_F32 = 0, 1
KFH_OUTGOING, KFH_INCOMING = 0, 1
KFH_STAGE_IN, KFH_STAGE_CORE, KFH_STAGE_OUT, KFH_STAGE_ALL = 1, 2, 4, 7
KFH_ARITH_BF16, KFH_ARITH_F32 = 0, 1

# name -> (restype, argtypes); mirrors include/kfold_hip.h one to one
_P = c_void_p
SIGNATURES: dict[str, tuple] = {
    "kfh_version": (c_int, []),
    "kfh_last_error": (c_char_p, []),
    "kfh_trimul_packed_bytes": (c_size_t, [c_int]),
    "kfh_trimul_pack": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int, _P, _P]),
    "kfh_trimul_workspace_bytes": (c_size_t, [c_int, c_int]),
    "kfh_trimul_workspace_bytes_batched": (c_size_t, [c_int, c_int, c_int]),
    "kfh_trimul_forward": (c_int, [_P, _P, _P, _P, _P, _P, c_size_t, c_int, c_int, c_int, c_int,
                                   c_float, c_int, _P]),
    "kfh_trimul_forward_stages": (c_int, [_P, _P, _P, _P, _P, _P, c_size_t, c_int, c_int, c_int, c_int,
                                          c_float, c_int, c_int, _P]),
    "kfh_triattn_forward_stages": (c_int, [_P, _P, _P, _P, _P, _P, c_size_t, c_int, c_int, c_int, c_int,
                                           c_int, c_float, c_int, c_int, _P]),
    "kfh_single_track_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int]),
    "kfh_single_track_forward": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_size_t, c_int, c_int, c_int, c_int, c_int,
                                         c_int, c_float, c_int, _P]),
    "kfh_pair_block_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    "kfh_pair_block_forward": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_size_t, c_int, c_int, c_int, c_int, c_int,
                                       c_float, c_int, _P]),
    "kfh_trimul_row_granule": (c_int, [c_int, c_int]),
    "kfh_trimul_forward_rows": (c_int, [_P, _P, _P, _P, _P, _P, c_size_t, c_int, c_int, c_int, c_int,
                                        c_float, c_int, c_int, c_int, c_int, _P]),
    "kfh_triattn_forward_rows": (c_int, [_P, _P, _P, _P, _P, _P, c_size_t, c_int, c_int, c_int, c_int,
                                         c_int, c_float, c_int, c_int, c_int, c_int, _P]),
    "kfh_triattn_packed_bytes": (c_size_t, [c_int, c_int]),
    "kfh_triattn_pack": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, _P, _P]),
    "kfh_triattn_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "kfh_triattn_workspace_bytes_batched": (c_size_t, [c_int, c_int, c_int, c_int]),
    "kfh_triattn_forward": (c_int, [_P, _P, _P, _P, _P, _P, c_size_t, c_int, c_int, c_int, c_int,
                                    c_int, c_float, c_int, _P]),
    "kfh_transition_packed_bytes": (c_size_t, [c_int, c_int]),
    "kfh_transition_pack": (c_int, [_P, _P, _P, _P, c_int, c_int, c_int, _P, _P]),
    "kfh_transition_workspace_bytes": (c_size_t, [c_longlong, c_int, c_int]),
    "kfh_transition_forward": (c_int, [_P, _P, _P, _P, _P, _P, c_size_t, c_longlong, c_int, c_int,
                                       c_float, c_int, _P]),
    "kfh_transition_static_scratch_bytes": (c_size_t, []),
    "kfh_transition_forward_static": (c_int, [_P, _P, _P, _P, _P, c_longlong, c_int, c_int, c_float, c_int, _P]),
    "kfh_bias_tiles_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "kfh_bias_tiles_from_dense": (c_int, [_P, c_int, _P, c_int, c_int, c_int, c_int, _P]),
    "kfh_pair_bias_packed_bytes": (c_size_t, [c_int, c_int]),
    "kfh_pair_bias_pack": (c_int, [_P, _P, _P, c_int, c_int, c_int, _P, _P]),
    "kfh_pair_bias_project": (c_int, [_P, _P, _P, c_int, c_int, c_int, c_int, c_float, c_int, _P]),
    "kfh_apb_packed_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "kfh_apb_pack": (c_int, [_P] * 14 + [c_int, c_int, c_int, c_int, c_int, _P, _P]),
    "kfh_apb_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int]),
    "kfh_apb_forward": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_size_t, c_int, c_int, c_int, c_int,
                                c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, _P]),
    "kfh_cross_apb_packed_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "kfh_cross_apb_pack": (c_int, [_P] * 20 + [c_int, c_int, c_int, c_int, c_int, _P, _P]),
    "kfh_cross_apb_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int, c_int]),
    "kfh_cross_apb_forward": (c_int, [_P, _P, _P, _P, _P, c_int, _P, _P, _P, _P, _P, c_size_t, c_int, c_int,
                                      c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, _P]),
    "kfh_parcae_packed_bytes": (c_size_t, [c_int]),
    "kfh_parcae_pack": (c_int, [_P, _P, _P, _P, _P, c_int, c_int, _P, _P]),
    "kfh_parcae_step": (c_int, [_P, _P, _P, _P, _P, c_longlong, c_int, c_float, c_int, _P]),
}

_lib = None


class KfoldHipError(RuntimeError):
    """A libkfold_hip.so entry point returned a non-zero status."""


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m kfold_amd.build` "
                "(the hip backend has no fallback path)")
        handle = ctypes.CDLL(str(LIB_PATH))
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(status: int) -> None:
    if status != 0:
        msg = lib().kfh_last_error().decode(errors="replace")
        raise KfoldHipError(f"libkfold_hip status {status}: {msg}")
