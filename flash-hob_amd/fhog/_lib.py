"""ctypes binding of ``libfhog_hip.so`` (C ABI in ``include/fhog_hip.h``).

The library is loaded from this directory.  It is never built implicitly at import time
on a machine with a GPU and there is no other implementation to fall back to: if the
shared object is missing, :func:`lib` raises.
"""
from __future__ import annotations

import ctypes
from ctypes import POINTER, Structure, c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_void_p
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libfhog_hip.so"

DTYPE_BF16, DTYPE_FP32, DTYPE_FP16 = 0, 1, 2
IMPL_AUTO, IMPL_FP32, IMPL_BF16 = 0, 1, 2
MASK_NONE, MASK_TOP_LEFT, MASK_BOTTOM_RIGHT = 0, 1, 2
PASS_D, PASS_DD, PASS_B, PASS_DQ_DDO, PASS_DK_DV, PASS_DD_B, PASS_B_DDO, PASS_DQ, PASS_DD_B_DDO, PASS_STAGE1 = range(10)
SCHEDULE_FOUR_PASS, SCHEDULE_FUSED_STATS, SCHEDULE_DDO_EARLY, SCHEDULE_THREE_SWEEP = range(4)
ABI_VERSION = 5
STATIC_WS_BYTES = 16 << 20   # of a default build; `lib().fhog_static_ws_bytes()` tells what the loaded library holds

ERROR_NAMES = {
    -1: "FHOG_E_NULL", -2: "FHOG_E_SHAPE", -3: "FHOG_E_DTYPE", -4: "FHOG_E_STRIDE", -5: "FHOG_E_ALIGN",
    -6: "FHOG_E_CAUSAL", -7: "FHOG_E_PASS", -8: "FHOG_E_LAUNCH", -9: "FHOG_E_SCALE", -10: "FHOG_E_IMPL",
    -11: "FHOG_E_SCHEDULE",
}


class BwdBwdArgs(Structure):
    """Mirror of ``fhog_bwdbwd_args``."""
    _fields_ = [
        ("q", c_void_p), ("k", c_void_p), ("v", c_void_p), ("o", c_void_p), ("dO", c_void_p),
        ("ddq", c_void_p), ("ddk", c_void_p), ("ddv", c_void_p), ("lse", c_void_p),
        ("dq2", c_void_p), ("dk2", c_void_p), ("dv2", c_void_p), ("ddo", c_void_p), ("ws", c_void_p),
        ("batch", c_int64), ("n_q", c_int64), ("n_k", c_int64), ("d", c_int64),
        ("stride_qb", c_int64), ("stride_qn", c_int64), ("stride_kb", c_int64), ("stride_kn", c_int64),
        ("scale", c_float), ("dtype", c_int32), ("causal", c_int32), ("impl", c_int32), ("schedule", c_int32),
        ("window", c_int64), ("ws_bytes", c_int64),
    ]


class AttnArgs(Structure):
    """Mirror of ``fhog_attn_args``."""
    _fields_ = [
        ("q", c_void_p), ("k", c_void_p), ("v", c_void_p), ("o", c_void_p), ("lse", c_void_p),
        ("dO", c_void_p), ("dq", c_void_p), ("dk", c_void_p), ("dv", c_void_p), ("ws", c_void_p),
        ("batch", c_int64), ("n_q", c_int64), ("n_k", c_int64), ("d", c_int64),
        ("stride_qb", c_int64), ("stride_qn", c_int64), ("stride_kb", c_int64), ("stride_kn", c_int64),
        ("scale", c_float), ("dtype", c_int32), ("causal", c_int32), ("window", c_int32),
    ]


class FhogError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"{ERROR_NAMES.get(code, code)}: {message}")
        self.code = code


_LIB = None


def lib() -> ctypes.CDLL:
    """Load (once) and return the shared library; raise if it is not there."""
    global _LIB
    if _LIB is not None:
        return _LIB
    if not LIB_PATH.exists():
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python flash-hob_amd/fhog/build.py` "
            "(hipcc, gfx950). There is no fallback implementation.")
    L = ctypes.CDLL(str(LIB_PATH))
    L.fhog_abi_version.restype = c_int
    L.fhog_abi_version.argtypes = []
    L.fhog_bwdbwd_workspace_bytes.restype = c_size_t
    L.fhog_bwdbwd_workspace_bytes.argtypes = [c_int64, c_int64]
    L.fhog_bwdbwd_workspace_hint.restype = c_size_t
    L.fhog_bwdbwd_workspace_hint.argtypes = [POINTER(BwdBwdArgs)]
    L.fhog_validate.restype = c_int
    L.fhog_validate.argtypes = [POINTER(BwdBwdArgs)]
    L.fhog_select_impl.restype = c_int
    L.fhog_select_impl.argtypes = [POINTER(BwdBwdArgs)]
    L.fhog_bwdbwd.restype = c_int
    L.fhog_bwdbwd.argtypes = [POINTER(BwdBwdArgs), c_void_p]
    L.fhog_bwdbwd_static_ws.restype = c_int
    L.fhog_bwdbwd_static_ws.argtypes = [POINTER(BwdBwdArgs), c_void_p]
    L.fhog_static_ws_bytes.restype = c_size_t
    L.fhog_static_ws_bytes.argtypes = []
    L.fhog_bwdbwd_pass.restype = c_int
    L.fhog_bwdbwd_pass.argtypes = [POINTER(BwdBwdArgs), c_int, c_void_p]
    L.fhog_last_error.restype = c_char_p
    L.fhog_last_error.argtypes = []
    L.fhog_bwdbwd_args_size.restype = c_size_t
    L.fhog_bwdbwd_args_size.argtypes = []
    L.fhog_attn_args_size.restype = c_size_t
    L.fhog_attn_args_size.argtypes = []
    L.fhog_attn_validate.restype = c_int
    L.fhog_attn_validate.argtypes = [POINTER(AttnArgs), c_int]
    L.fhog_attn_fwd.restype = c_int
    L.fhog_attn_fwd.argtypes = [POINTER(AttnArgs), c_void_p]
    L.fhog_attn_bwd.restype = c_int
    L.fhog_attn_bwd.argtypes = [POINTER(AttnArgs), c_void_p]
    L.fhog_probe_mfma_rate.restype = c_int
    L.fhog_probe_mfma_rate.argtypes = [c_void_p, c_int, c_int, c_int, POINTER(ctypes.c_double), c_void_p]
    if L.fhog_attn_args_size() != ctypes.sizeof(AttnArgs):
        raise RuntimeError("fhog_attn_args layout differs between libfhog_hip.so and the ctypes mirror")
    if L.fhog_bwdbwd_args_size() != ctypes.sizeof(BwdBwdArgs):
        raise RuntimeError("fhog_bwdbwd_args layout differs between libfhog_hip.so and the ctypes mirror")
    if L.fhog_abi_version() != ABI_VERSION:
        raise RuntimeError(f"libfhog_hip.so ABI {L.fhog_abi_version()} != binding {ABI_VERSION}")
    _LIB = L
    return L


def check(rc: int) -> None:
    if rc != 0:
        raise FhogError(rc, lib().fhog_last_error().decode())
