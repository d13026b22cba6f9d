"""
ctypes binding of ``librtn_native_lstm2.so`` (C ABI declared in ``include/rtn_native_lstm2.h``).

The library is the only implementation: there is no fallback.  If it has not been built,
:func:`load` raises and says how to build it.
"""

from __future__ import annotations

import ctypes
import os
import threading
from typing import Optional

from . import build as _build

RTN_OK = 0
RTN_ERR_SHAPE = 1
RTN_ERR_RANGE = 2
RTN_ERR_ARG = 3
RTN_ERR_WORKSPACE = 4
RTN_ERR_HIP = 5
RTN_ERR_UNSUPPORTED = 6
RTN_ERR_ABORTED = 7

DTYPE_F32 = 0
DTYPE_BF16 = 1

MODE_AUTO = 0
MODE_PERSISTENT = 1
MODE_GRAPH = 2
MODE_STEPWISE = 3
# The ABI version the structs and argument lists below were written for (rtn_native_lstm2_abi_version()).
EXPECTED_ABI = 13

MODES = {"auto": MODE_AUTO, "persistent": MODE_PERSISTENT, "graph": MODE_GRAPH, "stepwise": MODE_STEPWISE}

# every symbol include/rtn_native_lstm2.h declares
SYMBOLS = (
    "rtn_native_lstm2_fwd",
    "rtn_native_lstm2_fwd_workspace_bytes",
    "rtn_native_lstm2_fwd_static",
    "rtn_native_lstm2_fwd_status",
    "rtn_native_lstm2_fwd_multi",
    "rtn_native_lstm2_fwd_multi_workspace_bytes",
    "rtn_native_lstm2_fwd_multi_status",
    "rtn_handover_latency_probe",
    "rtn_mfma_sequence_probe",
    "rtn_mfma_issue_probe",
    "rtn_native_lstm2_bwd",
    "rtn_native_lstm2_bwd_workspace_bytes",
    "rtn_native_lstm2_bwd_multi",
    "rtn_native_lstm2_bwd_multi_workspace_bytes",
    "rtn_lstm_generic_base_fwd",
    "rtn_lstm_generic_base_fwd_workspace_bytes",
    "rtn_lstm_generic_base_bwd",
    "rtn_lstm_generic_base_bwd_workspace_bytes",
    "rtn_lstm_low_mem_fwd",
    "rtn_lstm_low_mem_fwd_workspace_bytes",
    "rtn_lstm_low_mem_bwd",
    "rtn_lstm_low_mem_bwd_workspace_bytes",
    "rtn_native_lstm2_last_output",
    "rtn_last_error",
    "rtn_native_lstm2_describe_plan",
    "rtn_native_lstm2_describe_multi_plan",
    "rtn_graph_cache_stats",
    "rtn_native_lstm2_capture_report",
    "rtn_native_lstm2_bwd_plan_text",
    "rtn_native_lstm2_reload_env",
    "rtn_native_lstm2_abi_version",
)



class Lstm2Call(ctypes.Structure):
    """``rtn_lstm2_call``: the arguments of one op call inside ``rtn_native_lstm2_fwd_multi``."""

    _fields_ = [
        ("X", ctypes.c_void_p),
        ("W", ctypes.c_void_p),
        ("y0", ctypes.c_void_p),
        ("c0", ctypes.c_void_p),
        ("i", ctypes.c_void_p),
        ("start", ctypes.c_int32),
        ("step", ctypes.c_int32),
        ("Y", ctypes.c_void_p),
        ("C", ctypes.c_void_p),
        ("H", ctypes.c_void_p),
        ("d", ctypes.c_void_p),
        ("ldX", ctypes.c_int64),  # row pitch of X in elements, 0 = contiguous (4n)
        ("ldY", ctypes.c_int64),  # row pitch of Y in elements, 0 = contiguous (n)
    ]


class Lstm2BwdCall(ctypes.Structure):
    """``rtn_lstm2_bwd_call``: the arguments of one gradient call inside ``rtn_native_lstm2_bwd_multi``."""

    _fields_ = [
        ("W", ctypes.c_void_p),
        ("y0", ctypes.c_void_p),
        ("c0", ctypes.c_void_p),
        ("i", ctypes.c_void_p),
        ("start", ctypes.c_int32),
        ("step", ctypes.c_int32),
        ("Y", ctypes.c_void_p),
        ("C", ctypes.c_void_p),
        ("H", ctypes.c_void_p),
        ("DY", ctypes.c_void_p),
        ("Dd", ctypes.c_void_p),
        ("DX", ctypes.c_void_p),
        ("DW", ctypes.c_void_p),
        ("Dy0", ctypes.c_void_p),
        ("Dc0", ctypes.c_void_p),
        ("ldY", ctypes.c_int64),  # row pitch of Y in elements, 0 = contiguous (n)
        ("ldDY", ctypes.c_int64),  # row pitch of DY in elements, 0 = contiguous (n)
        ("ldDX", ctypes.c_int64),  # row pitch of DX in elements, 0 = contiguous (4n)
    ]


_lock = threading.RLock()
_lib: Optional[ctypes.CDLL] = None


class NativeLibraryMissing(RuntimeError):
    """The HIP library has not been built."""


class NativeLibraryMismatch(RuntimeError):
    """The built library reports another ABI version than this binding was written for (a stale build)."""


def load() -> ctypes.CDLL:
    """Load the built library (once per process). Never builds, never falls back."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = os.environ.get("RTN_NATIVE_LSTM2_LIB") or _build.LIB_PATH  # override: an instrumented build
        if not os.path.exists(path):
            raise NativeLibraryMissing(
                "%s not found. Build it with `python -m returnn_amd.build` (needs hipcc; "
                "cross-compiles for gfx950 without a GPU)." % path
            )
        lib = ctypes.CDLL(path)
        lib.rtn_native_lstm2_abi_version.restype = ctypes.c_int
        lib.rtn_native_lstm2_abi_version.argtypes = []
        abi = int(lib.rtn_native_lstm2_abi_version())
        if abi != EXPECTED_ABI:
            # calling on with other struct layouts or argument lists would write through wrong device pointers
            raise NativeLibraryMismatch(
                "%s reports ABI version %i, this binding is written for %i: rebuild it with `python -m returnn_amd.build`"
                % (path, abi, EXPECTED_ABI)
            )
        vp, i32, i64, sz = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_size_t
        lib.rtn_native_lstm2_fwd.restype = ctypes.c_int
        lib.rtn_native_lstm2_fwd.argtypes = [vp, vp, vp, vp, vp, i32, i32, vp, vp, vp, vp, i64, i32, i32, i32, i32, vp, sz, vp]
        lib.rtn_native_lstm2_fwd_static.restype = ctypes.c_int
        lib.rtn_native_lstm2_fwd_static.argtypes = [vp, vp, vp, vp, vp, i32, i32, vp, vp, vp, vp, i64, i32, i32, i32, i32, vp]
        lib.rtn_native_lstm2_fwd_workspace_bytes.restype = sz
        lib.rtn_native_lstm2_fwd_workspace_bytes.argtypes = [i64, i32, i32, i32, i32]
        lib.rtn_native_lstm2_fwd_status.restype = ctypes.c_int
        lib.rtn_native_lstm2_fwd_status.argtypes = [vp, vp]
        lib.rtn_native_lstm2_fwd_multi.restype = ctypes.c_int
        lib.rtn_native_lstm2_fwd_multi.argtypes = [ctypes.POINTER(Lstm2Call), i32, i64, i32, i32, i32, i32, vp, sz, vp]
        lib.rtn_native_lstm2_fwd_multi_workspace_bytes.restype = sz
        lib.rtn_native_lstm2_fwd_multi_workspace_bytes.argtypes = [i32, i64, i32, i32, i32, i32]
        lib.rtn_native_lstm2_fwd_multi_status.restype = ctypes.c_int
        lib.rtn_native_lstm2_fwd_multi_status.argtypes = [vp, i32, i64, i32, i32, i32, i32, vp]
        lib.rtn_native_lstm2_bwd.restype = ctypes.c_int
        lib.rtn_native_lstm2_bwd.argtypes = [vp, vp, vp, vp, i32, i32, vp, vp, vp, vp, vp, vp, vp, vp, vp, i64, i32, i32, i32, vp, sz, vp]
        lib.rtn_native_lstm2_bwd_workspace_bytes.restype = sz
        lib.rtn_native_lstm2_bwd_workspace_bytes.argtypes = [i64, i32, i32, i32]
        lib.rtn_native_lstm2_bwd_multi.restype = ctypes.c_int
        lib.rtn_native_lstm2_bwd_multi.argtypes = [ctypes.POINTER(Lstm2BwdCall), i32, i64, i32, i32, i32, vp, sz, vp]
        lib.rtn_native_lstm2_bwd_multi_workspace_bytes.restype = sz
        lib.rtn_native_lstm2_bwd_multi_workspace_bytes.argtypes = [i32, i64, i32, i32, i32]
        lib.rtn_lstm_generic_base_fwd.restype = ctypes.c_int
        lib.rtn_lstm_generic_base_fwd.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i32, i32, i32, i32, vp, sz, vp]
        lib.rtn_lstm_generic_base_fwd_workspace_bytes.restype = sz
        lib.rtn_lstm_generic_base_fwd_workspace_bytes.argtypes = [i64, i32, i32, i32, i32]
        lib.rtn_lstm_generic_base_bwd.restype = ctypes.c_int
        lib.rtn_lstm_generic_base_bwd.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, i64, i32, i32, i32, vp, sz, vp]
        lib.rtn_lstm_generic_base_bwd_workspace_bytes.restype = sz
        lib.rtn_lstm_generic_base_bwd_workspace_bytes.argtypes = [i64, i32, i32, i32]
        lib.rtn_lstm_low_mem_fwd.restype = ctypes.c_int
        lib.rtn_lstm_low_mem_fwd.argtypes = [vp, vp, vp, vp, vp, vp, i32, i32, vp, vp, vp, i64, i32, i32, i32, i32, i32, vp, sz, vp]
        lib.rtn_lstm_low_mem_fwd_workspace_bytes.restype = sz
        lib.rtn_lstm_low_mem_fwd_workspace_bytes.argtypes = [i64, i32, i32, i32, i32, i32]
        lib.rtn_lstm_low_mem_bwd.restype = ctypes.c_int
        lib.rtn_lstm_low_mem_bwd.argtypes = [vp] * 6 + [i32, i32] + [vp] * 9 + [i64, i32, i32, i32, i32, vp, sz, vp]
        lib.rtn_lstm_low_mem_bwd_workspace_bytes.restype = sz
        lib.rtn_lstm_low_mem_bwd_workspace_bytes.argtypes = [i64, i32, i32, i32, i32]
        lib.rtn_native_lstm2_bwd_plan_text.restype = ctypes.c_char_p
        lib.rtn_native_lstm2_bwd_plan_text.argtypes = []
        lib.rtn_native_lstm2_capture_report.restype = ctypes.c_char_p
        lib.rtn_native_lstm2_capture_report.argtypes = []
        lib.rtn_graph_cache_stats.restype = ctypes.c_int
        lib.rtn_graph_cache_stats.argtypes = [ctypes.POINTER(ctypes.c_int64), i32]
        lib.rtn_mfma_sequence_probe.restype = ctypes.c_int
        lib.rtn_mfma_sequence_probe.argtypes = [i32, i64, i32, i32, i32, i32, vp, sz, vp]
        lib.rtn_mfma_issue_probe.restype = ctypes.c_int
        lib.rtn_mfma_issue_probe.argtypes = [i32, i64, i32, i32, i32, i32, vp, sz, vp]
        lib.rtn_handover_latency_probe.restype = ctypes.c_int
        lib.rtn_handover_latency_probe.argtypes = [vp, sz, i32, vp]
        lib.rtn_native_lstm2_last_output.restype = ctypes.c_int
        lib.rtn_native_lstm2_last_output.argtypes = [vp, vp, vp, i32, i32, vp, i64, i32, i32, i32, i64, vp]
        lib.rtn_last_error.restype = ctypes.c_char_p
        lib.rtn_last_error.argtypes = []
        lib.rtn_native_lstm2_describe_plan.restype = ctypes.c_char_p
        lib.rtn_native_lstm2_describe_plan.argtypes = [i64, i32, i32, i32, i32]
        lib.rtn_native_lstm2_describe_multi_plan.restype = ctypes.c_char_p
        lib.rtn_native_lstm2_describe_multi_plan.argtypes = [i32, i64, i32, i32, i32, i32]
        lib.rtn_native_lstm2_reload_env.restype = None
        lib.rtn_native_lstm2_reload_env.argtypes = []
        _lib = lib
        return lib


def reload_env() -> None:
    """Make the library read its ``RTN_LSTM2_*`` environment variables again (it reads them once, at first use).  Does
    nothing while the library is not loaded: its first use will read the environment as it is then."""
    with _lock:
        lib = _lib
    if lib is not None:
        lib.rtn_native_lstm2_reload_env()


def last_error() -> str:
    return load().rtn_last_error().decode("utf8", "replace")


def check(rc: int) -> None:
    """Turn a status code of the C ABI into the exception the reference's wrapper would raise
    (TORCH_CHECK -> RuntimeError, returnn/native_op.cpp:660)."""
    if rc != RTN_OK:
        raise RuntimeError(last_error() or ("NativeLstm2: error code %i" % rc))


def bwd_plan_text() -> str:
    return load().rtn_native_lstm2_bwd_plan_text().decode("utf8", "replace")


def capture_report() -> str:
    return load().rtn_native_lstm2_capture_report().decode("utf8", "replace")


def graph_cache_stats() -> dict:
    """Counters of the library-owned graph cache: kept, retiring, built, retargeted, destroyed."""
    out = (ctypes.c_int64 * 5)()
    check(load().rtn_graph_cache_stats(out, 5))
    return dict(zip(("kept", "retiring", "built", "retargeted", "destroyed"), (int(v) for v in out)))


def describe_plan(T: int, B: int, n: int, dtype: int, mode: int) -> str:
    return load().rtn_native_lstm2_describe_plan(T, B, n, dtype, mode).decode("utf8", "replace")


def describe_multi_plan(count: int, T: int, B: int, n: int, dtype: int, mode: int) -> str:
    return load().rtn_native_lstm2_describe_multi_plan(count, T, B, n, dtype, mode).decode("utf8", "replace")


def workspace_bytes(T: int, B: int, n: int, dtype: int, mode: int) -> int:
    return int(load().rtn_native_lstm2_fwd_workspace_bytes(T, B, n, dtype, mode))
