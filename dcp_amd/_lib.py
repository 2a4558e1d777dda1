"""ctypes binding of libdcp_hip.so.

The library is the only compute backend: if it is missing or fails to load,
every operator raises instead of falling back to another implementation.
"""

from __future__ import annotations

import ctypes
import os
import threading
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p
from pathlib import Path

LIB_PATH = Path(os.environ.get("DCP_LIB_PATH", Path(__file__).resolve().parent / "libdcp_hip.so"))

_P = c_void_p
_I = c_int
_L = c_int64
_F = c_float

# symbol -> argument types (all return int unless noted)
SIGNATURES = {
    "dcp_version": [],
    "dcp_last_error": [],
    "dcp_profile_enable": [_I],
    "dcp_profile_report": [c_char_p, c_size_t],
    "dcp_fused_copy_varlen": [_P, _P, _P, _P, _P, _P, _P, _I, _L, _I, _P],
    "dcp_fused_copy_varlen_dkv": [_P, _P, _P, _I, _I, _I, _I, _P],
    "dcp_fused_copy_varlen_lse": [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P],
    "dcp_update_out_lse": [_P, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _L, _L, _L, _L, _L, _L, _I, _I, _I, _P],
    "dcp_blockwise_sum": [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _L, _I, _P],
    "dcp_attn_fwd": [_P, _P, _P, _P, _P, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _L, _L, _I, _F, _I, _P, c_size_t, _P],
    "dcp_attn_fwd_workspace_bytes": [],
    "dcp_attn_bwd": [_P] * 10 + [c_size_t] + [_P] * 3 + [_I] + [_P] * 6 + [_I] * 7 + [_L] * 4 + [_I, _F, _I, _P],
    "dcp_attn_fwd_strided": [_P, _P, _P, _P, _P, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I] + [_L] * 6
                            + [_I, _F, _I, _P, c_size_t, _P],
    "dcp_attn_bwd_strided": [_P] * 10 + [c_size_t] + [_P] * 3 + [_I] + [_P] * 6 + [_I] * 7 + [_L] * 10 + [_F, _I, _P],
    "dcp_attn_bwd_workspace_bytes_kv": [_I, _I, _L, _I, _I, _I],
    "dcp_attn_bwd_workspace_bytes": [_I, _I, _I, _I, _I],
    "dcp_attn_bwd_static": [_P] * 9 + [_P] * 3 + [_I] + [_P] * 6 + [_I] * 7 + [_L] * 4 + [_I, _F, _I, _P],
    "dcp_attn_bwd_static_scratch_bytes": [],
    "dcp_attn_bwd_select": [_I],
    "dcp_greedy_stage_selection": [_I, _P, _I, _P, _P, _I, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _P, _P, _P, _P, _L, _P, _P, _P],
}

_lock = threading.Lock()
_lib = None


class DcpHipError(RuntimeError):
    """The HIP library is unavailable or rejected a call."""


def load():
    """Return the loaded library (loads it on first use)."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not LIB_PATH.exists():
            raise DcpHipError(
                f"{LIB_PATH} is not built; run `python -m dcp_amd.build` "
                "(there is no fallback implementation)"
            )
        # torch bundles its own HIP runtime (same soname as the system one).
        # It must be in the process before this library is, so that both bind
        # to one runtime; two runtimes in one process do not share a device.
        import torch  # noqa: F401

        lib = ctypes.CDLL(str(LIB_PATH))
        for name, argtypes in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = {"dcp_last_error": c_char_p, "dcp_attn_bwd_workspace_bytes": c_size_t,
                          "dcp_attn_fwd_workspace_bytes": c_size_t,
                          "dcp_attn_bwd_static_scratch_bytes": c_size_t,
                          "dcp_attn_bwd_workspace_bytes_kv": c_size_t}.get(name, c_int)
        _lib = lib
    return _lib


def profile_enable(on: bool) -> None:
    load().dcp_profile_enable(1 if on else 0)


def profile_report() -> dict:
    """``{kernel name: (launches, total milliseconds)}`` of the launches made
    while profiling was enabled; clears the record."""
    buf = ctypes.create_string_buffer(1 << 16)
    status = load().dcp_profile_report(buf, len(buf))
    if status != 0:
        raise DcpHipError("dcp_profile_report: buffer too small")
    out = {}
    for line in buf.value.decode().splitlines():
        name, count, total = line.rsplit(" ", 2)
        out[name] = (int(count), float(total))
    return out


def last_error() -> str:
    return load().dcp_last_error().decode(errors="replace")


def call(name: str, *args) -> None:
    """Call an entry point; a nonzero status becomes an exception carrying the
    library's message: ``ValueError`` for unsupported types (status 2),
    ``AssertionError`` for argument preconditions (status 1), as the reference
    operators raise for the same conditions."""
    status = getattr(load(), name)(*args)
    if status == 0:
        return
    message = f"{name}: {last_error()}"
    if status == 2:
        raise ValueError(message)
    if status == 1:
        raise AssertionError(message)
    raise DcpHipError(message)
