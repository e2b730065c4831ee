"""ctypes binding of libfox_attn.so (see include/fox_attn.h for the ABI).

The library is loaded lazily and exactly once.  There is no fallback: if the
shared object is missing or a call fails, a ``RuntimeError`` is raised.
"""
from __future__ import annotations

import ctypes as C
import threading
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent.parent / "_lib" / "libfox_attn.so"

DTYPE_BF16 = 0
DTYPE_FP16 = 1
DTYPE_FP32 = 2  # gate logits only


class View(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("stride_b", C.c_int64), ("stride_h", C.c_int64), ("stride_t", C.c_int64)]


class Dims(C.Structure):
    _fields_ = [("B", C.c_int32), ("H", C.c_int32), ("M", C.c_int32), ("N", C.c_int32), ("D", C.c_int32),
                ("dtype", C.c_int32)]


class FwdArgs(C.Structure):
    _fields_ = [
        ("dims", Dims),
        ("q", View), ("k", View), ("v", View), ("o", View),
        ("log_lambda", C.c_void_p),
        ("lse", C.c_void_p),
        ("seq_start", C.c_void_p),
        ("threshold", C.c_void_p),
        ("sm_scale", C.c_float),
        ("first_block", C.c_void_p),
        ("workspace", C.c_void_p),
        ("workspace_bytes", C.c_int64),
    ]


class BwdArgs(C.Structure):
    _fields_ = [
        ("dims", Dims),
        ("q", View), ("k", View), ("v", View), ("o", View), ("d_o", View),
        ("dq", View), ("dk", View), ("dv", View),
        ("log_lambda", C.c_void_p),
        ("lse", C.c_void_p),
        ("seq_start", C.c_void_p),
        ("threshold", C.c_void_p),
        ("sm_scale", C.c_float),
        ("delta", C.c_void_p),
        ("drow", C.c_void_p),
        ("dlog_lambda", C.c_void_p),
        ("dlog_fgate", C.c_void_p),
        ("dlog_fgate_stride_b", C.c_int64), ("dlog_fgate_stride_h", C.c_int64), ("dlog_fgate_stride_n", C.c_int64),
        ("q_first_block", C.c_void_p),
        ("kv_end_row", C.c_void_p),
    ]


class ShiftArgs(C.Structure):
    _fields_ = [
        ("B", C.c_int32), ("T", C.c_int32), ("H", C.c_int32), ("D", C.c_int32),
        ("dtype", C.c_int32),
        ("x", C.c_void_p),
        ("x_stride_b", C.c_int64), ("x_stride_t", C.c_int64), ("x_stride_h", C.c_int64),
        ("prev_weight", C.c_void_p),
        ("curr_weight", C.c_void_p),
        ("w_stride_b", C.c_int64), ("w_stride_t", C.c_int64), ("w_stride_h", C.c_int64),
        ("out", C.c_void_p),
        ("dout", C.c_void_p),
        ("dx", C.c_void_p),
        ("dprev_weight", C.c_void_p),
        ("dcurr_weight", C.c_void_p),
    ]


ACT_SIGMOID = 0
ACT_SWISH = 1
ACT_NONE = 2


class NormGateArgs(C.Structure):
    _fields_ = [
        ("rows", C.c_int64),
        ("G", C.c_int32), ("D", C.c_int32),
        ("dtype", C.c_int32),
        ("activation", C.c_int32),
        ("eps", C.c_float),
        ("x", C.c_void_p), ("x_stride_row", C.c_int64),
        ("g", C.c_void_p), ("g_stride_row", C.c_int64),
        ("weight", C.c_void_p),
        ("y", C.c_void_p), ("y_stride_row", C.c_int64),
        ("rstd", C.c_void_p),
        ("dy", C.c_void_p), ("dy_stride_row", C.c_int64),
        ("dx", C.c_void_p), ("dx_stride_row", C.c_int64),
        ("dg", C.c_void_p), ("dg_stride_row", C.c_int64),
        ("dweight", C.c_void_p),
        ("workspace", C.c_void_p),
    ]


class FwdEpilogue(C.Structure):
    _fields_ = [
        ("gate", View), ("y", View),
        ("weight", C.c_void_p),
        ("rstd", C.c_void_p),
        ("eps", C.c_float),
        ("activation", C.c_int32),
    ]


# every symbol include/fox_attn.h declares: name -> (restype, argtypes)
SIGNATURES = {
    "fox_version": (C.c_int, []),
    "fox_last_error": (C.c_char_p, []),
    "fox_set_acp_light_limit": (C.c_int32, [C.c_int32]),
    "fox_set_stream_min_kv_bytes": (C.c_int64, [C.c_int64]),
    "fox_probe_mfma": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_void_p]),
    "fox_tile_config": (C.c_int, [C.c_int32] + [C.POINTER(C.c_int32)] * 4),
    "fox_cumsum_fwd": (C.c_int, [C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32,
                                 C.c_int32, C.c_void_p]),
    "fox_cumsum_bwd": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_void_p, C.c_int32, C.c_int32, C.c_int32,
                                 C.c_void_p]),
    "fox_gate_cumsum_fwd": (C.c_int, [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p,
                                      C.c_int32, C.c_int32, C.c_int32, C.c_void_p]),
    "fox_gate_cumsum_bwd": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p,
                                      C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_int32, C.c_int32, C.c_void_p]),
    "fox_auto_threshold": (C.c_int, [C.POINTER(Dims), C.POINTER(View), C.POINTER(View), C.c_float, C.c_void_p, C.c_void_p,
                                     C.c_void_p]),
    "fox_attn_fwd": (C.c_int, [C.POINTER(FwdArgs), C.c_void_p]),
    "fox_attn_fwd_noalloc": (C.c_int, [C.POINTER(FwdArgs), C.c_void_p]),
    "fox_attn_fwd_norm_gate": (C.c_int, [C.POINTER(FwdArgs), C.POINTER(FwdEpilogue), C.c_void_p]),
    "fox_attn_fwd_workspace_bytes": (C.c_int, [C.POINTER(Dims), C.POINTER(C.c_int64)]),
    "fox_attn_bwd_delta": (C.c_int, [C.POINTER(BwdArgs), C.c_void_p]),
    "fox_attn_bwd_dkdv": (C.c_int, [C.POINTER(BwdArgs), C.c_void_p]),
    "fox_attn_bwd_dq": (C.c_int, [C.POINTER(BwdArgs), C.c_void_p]),
    "fox_attn_bwd": (C.c_int, [C.POINTER(BwdArgs), C.c_void_p]),
    "fox_norm_gate_fwd": (C.c_int, [C.POINTER(NormGateArgs), C.c_void_p]),
    "fox_norm_gate_bwd": (C.c_int, [C.POINTER(NormGateArgs), C.c_void_p]),
    "fox_norm_gate_workspace_bytes": (C.c_int, [C.c_int64, C.c_int32, C.c_int32, C.POINTER(C.c_int64)]),
    "fox_token_shift_fwd": (C.c_int, [C.POINTER(ShiftArgs), C.c_void_p]),
    "fox_token_shift_bwd": (C.c_int, [C.POINTER(ShiftArgs), C.c_void_p]),
}

_lib = None
_lock = threading.Lock()


def load() -> C.CDLL:
    """Load libfox_attn.so and bind every declared symbol."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not LIB_PATH.exists():
                raise RuntimeError(
                    f"{LIB_PATH} is missing: build it with `python forgetting-transformer_amd/build.py` "
                    "(there is no fallback implementation)")
            lib = C.CDLL(str(LIB_PATH))
            for name, (restype, argtypes) in SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype = restype
                fn.argtypes = argtypes
            _lib = lib
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().fox_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed (code {rc}): {msg}")


def tile_config(head_dim: int):
    """(block_m, block_n, kv_block_n, kv_block_m) for a head dim."""
    vals = [C.c_int32() for _ in range(4)]
    check(load().fox_tile_config(head_dim, *[C.byref(v) for v in vals]), "fox_tile_config")
    return tuple(v.value for v in vals)
