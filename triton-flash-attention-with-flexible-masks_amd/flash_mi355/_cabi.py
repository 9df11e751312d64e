"""ctypes binding of libflash_mi355.so (the C ABI declared in include/flash_mi355.h).

The library is loaded from this package directory only; there is no fallback
implementation.  If it is missing, ``lib()`` raises and every operator call fails.
"""
from __future__ import annotations

import ctypes
from ctypes import POINTER, Structure, c_char_p, c_float, c_int, c_int32, c_int64, c_uint64, c_void_p
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libflash_mi355.so"

FA_ABI_VERSION = 7
FA_SCORE_MODE0_NOPE = 0
FA_SCORE_MODE1_DOC = 1
FA_SCORE_MODE2_BLOCK = 2
FA_MASK_BLOCK = 64
FA_DTYPE_BF16 = 0
FA_DTYPE_FP16 = 1
FA_DTYPE_FP32 = 2
FA_IDTYPE_I32 = 0
FA_IDTYPE_I64 = 1
FA_FLAG_DQ_DELTA = 1
FA_FLAG_DEBUG_NO_PAIR_WAIT = 0x100
FA_STATIC_WS_BYTES = 32 << 20

# every symbol include/flash_mi355.h declares
EXPORTS = (
    "fa_version", "fa_params_size", "fa_error_string", "fa_last_hip_error", "fa_validate",
    "fa_workspace_bytes", "fa_workspace_plan_bytes", "fa_mask_plan", "fa_fwd", "fa_bwd_delta", "fa_bwd_dkdv", "fa_bwd_dq",
    "fa_mask_dump", "fa_fwd_static", "fa_workspace_scratch_bytes", "fa_pair_wait_expired",
)


class FaParams(Structure):
    """Mirror of ``struct fa_params``; field order and types must match the header."""
    _fields_ = [
        ("q", c_void_p), ("k", c_void_p), ("v", c_void_p), ("o", c_void_p), ("lse", c_void_p),
        ("dout", c_void_p), ("dq", c_void_p), ("dk", c_void_p), ("dv", c_void_p), ("delta", c_void_p),
        ("eq", c_void_p), ("ek", c_void_p),
        ("workspace", c_void_p), ("workspace_bytes", c_uint64),
        ("q_stride", c_int64 * 4), ("k_stride", c_int64 * 4), ("v_stride", c_int64 * 4), ("o_stride", c_int64 * 4),
        ("do_stride", c_int64 * 4), ("dq_stride", c_int64 * 4), ("dk_stride", c_int64 * 4), ("dv_stride", c_int64 * 4),
        ("eq_stride", c_int64 * 3), ("ek_stride", c_int64 * 3),
        ("B", c_int32), ("H", c_int32), ("Hk", c_int32), ("M", c_int32), ("N", c_int32), ("D", c_int32),
        ("causal", c_int32), ("score_mode", c_int32), ("dtype", c_int32), ("id_dtype", c_int32),
        ("sm_scale", c_float), ("flags", c_int32), ("window", c_int32), ("prefix", c_int32),
        ("qpos", c_void_p), ("qpos_stride", c_int64),
        ("split_scratch", c_void_p), ("split_scratch_bytes", c_uint64),
    ]


_lib = None


class FlashMI355Error(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    """Load (once) and return the shared library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise FlashMI355Error(
            f"{LIB_PATH} is missing: build it with `python -m flash_mi355.build` "
            "(there is no fallback implementation)")
    L = ctypes.CDLL(str(LIB_PATH))
    L.fa_version.restype = c_int
    L.fa_params_size.restype = c_uint64
    L.fa_error_string.restype = c_char_p
    L.fa_error_string.argtypes = [c_int]
    L.fa_last_hip_error.restype = c_int
    L.fa_validate.restype = c_int
    L.fa_validate.argtypes = [POINTER(FaParams), c_int]
    L.fa_workspace_bytes.restype = c_uint64
    L.fa_workspace_bytes.argtypes = [POINTER(FaParams)]
    L.fa_workspace_plan_bytes.restype = c_uint64
    L.fa_workspace_plan_bytes.argtypes = [POINTER(FaParams)]
    L.fa_workspace_scratch_bytes.restype = c_uint64
    L.fa_workspace_scratch_bytes.argtypes = [POINTER(FaParams)]
    L.fa_pair_wait_expired.restype = c_int
    L.fa_pair_wait_expired.argtypes = [POINTER(c_uint64)]
    for name in ("fa_mask_plan", "fa_fwd", "fa_fwd_static", "fa_bwd_delta", "fa_bwd_dkdv", "fa_bwd_dq"):
        fn = getattr(L, name)
        fn.restype = c_int
        fn.argtypes = [POINTER(FaParams), c_void_p]
    L.fa_mask_dump.restype = c_int
    L.fa_mask_dump.argtypes = [POINTER(FaParams), c_void_p, c_void_p]
    if L.fa_version() != FA_ABI_VERSION:
        raise FlashMI355Error(f"ABI mismatch: library {L.fa_version()}, binding {FA_ABI_VERSION}")
    if L.fa_params_size() != ctypes.sizeof(FaParams):
        raise FlashMI355Error(
            f"fa_params size mismatch: library {L.fa_params_size()}, binding {ctypes.sizeof(FaParams)}")
    _lib = L
    return L


def check(rc: int, what: str) -> None:
    if rc != 0:
        L = lib()
        msg = L.fa_error_string(rc).decode()
        extra = f" (hipError {L.fa_last_hip_error()})" if rc == -9 else ""
        raise FlashMI355Error(f"{what}: {msg}{extra} [code {rc}]")
