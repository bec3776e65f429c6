"""ctypes binding of ``libkvax_amd.so`` (the C ABI declared in ``include/kvax_amd.h``).

There is no fallback: if the shared library is missing, every op raises ``KvaxNativeError``
telling the caller to build it (``python -m kvax_amd.csrc.build``).
"""
from __future__ import annotations

import ctypes as C
import os
from pathlib import Path

LIB_PATH = Path(os.environ.get("KVAX_AMD_LIB") or Path(__file__).resolve().parent / "libkvax_amd.so")
ABI_VERSION = 1
KVAX_MAX_MASKS = 4
KVAX_BF16, KVAX_F16 = 0, 1
KVAX_FA_DKDV_F32 = 1
KVAX_FA_SKIP_DELTA, KVAX_FA_SKIP_DQ, KVAX_FA_SKIP_DKDV = 16, 32, 64
KVAX_FA_FWD_WIDE = 128
KVAX_FA_FWD_STATIC_MAX_WORKSPACE = 8 << 20


class KvaxNativeError(RuntimeError):
    pass


class MaskDesc(C.Structure):
    _fields_ = [
        ("query_block_size", C.c_int32),
        ("kv_block_size", C.c_int32),
        ("kv_outer", C.c_int32),
        ("reserved", C.c_int32),
        ("lower", C.c_void_p),
        ("upper", C.c_void_p),
        ("lower_full", C.c_void_p),
        ("upper_full", C.c_void_p),
    ]


class FaArgs(C.Structure):
    """Mirror of ``kvax_fa_args`` (see include/kvax_amd.h for the meaning of each field)."""

    _fields_ = [
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p),
        ("out", C.c_void_p), ("lse", C.c_void_p),
        ("dout", C.c_void_p), ("dq", C.c_void_p), ("dk", C.c_void_p), ("dv", C.c_void_p),
        ("q_pos", C.c_void_p), ("q_seg", C.c_void_p), ("kv_pos", C.c_void_p), ("kv_seg", C.c_void_p),
        ("fwd_mask", C.c_void_p * 4), ("dq_mask", C.c_void_p * 4), ("dkdv_mask", C.c_void_p * 4),
        ("q_strides", C.c_int64 * 3), ("k_strides", C.c_int64 * 3), ("v_strides", C.c_int64 * 3),
        ("o_strides", C.c_int64 * 3), ("do_strides", C.c_int64 * 3), ("dq_strides", C.c_int64 * 3),
        ("dk_strides", C.c_int64 * 3), ("dv_strides", C.c_int64 * 3),
        ("batch", C.c_int32), ("q_len", C.c_int32), ("kv_len", C.c_int32),
        ("num_heads", C.c_int32), ("num_kv_heads", C.c_int32), ("head_dim", C.c_int32),
        ("fwd_query_block", C.c_int32), ("fwd_kv_block", C.c_int32),
        ("bwd_query_block", C.c_int32), ("bwd_kv_block", C.c_int32),
        ("dtype", C.c_int32), ("flags", C.c_int32),
        ("scale", C.c_float), ("reserved", C.c_int32),
    ]


_lib = None


def lib() -> C.CDLL:
    """Load the library once; raise loudly when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise KvaxNativeError(
            f"{LIB_PATH} not found: the HIP extension is not built. "
            "Run `python -m kvax_amd.csrc.build` (needs hipcc; no GPU required to compile)."
        )
    try:
        l = C.CDLL(str(LIB_PATH))
    except OSError as e:  # missing ROCm runtime etc.
        raise KvaxNativeError(f"cannot load {LIB_PATH}: {e}") from e
    l.kvax_abi_version.restype = C.c_int
    l.kvax_last_error.restype = C.c_char_p
    if l.kvax_abi_version() != ABI_VERSION:
        raise KvaxNativeError(
            f"{LIB_PATH} has ABI version {l.kvax_abi_version()}, expected {ABI_VERSION}: rebuild it"
        )
    l.kvax_mask_workspace_bytes.restype = C.c_size_t
    l.kvax_mask_workspace_bytes.argtypes = [C.c_int, C.c_int, C.c_int, C.POINTER(MaskDesc), C.c_int]
    l.kvax_mask_build.restype = C.c_int
    l.kvax_mask_build.argtypes = [
        C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
        C.POINTER(MaskDesc), C.c_int, C.c_void_p, C.c_size_t, C.c_void_p,
    ]
    for name in ("kvax_fa_fwd", "kvax_fa_bwd"):
        if hasattr(l, name):
            fn = getattr(l, name)
            fn.restype = C.c_int
            fn.argtypes = [C.POINTER(FaArgs), C.c_void_p, C.c_size_t, C.c_void_p]
    if hasattr(l, "kvax_fa_fwd_static"):
        l.kvax_fa_fwd_static.restype = C.c_int
        l.kvax_fa_fwd_static.argtypes = [C.POINTER(FaArgs), C.c_void_p]
    for name in ("kvax_fa_fwd_workspace_bytes", "kvax_fa_bwd_workspace_bytes"):
        if hasattr(l, name):
            fn = getattr(l, name)
            fn.restype = C.c_size_t
            fn.argtypes = [C.POINTER(FaArgs)]
    _lib = l
    return l


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = lib().kvax_last_error().decode(errors="replace")
        raise KvaxNativeError(f"{what} failed with code {rc}: {msg}")
