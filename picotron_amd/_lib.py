"""ctypes binding of libpicotron_amd.so (see include/picotron_amd.h for the contract).

The library is the product: there is no Python or torch fallback.  If it has not been built,
``lib()`` raises with the build command instead of computing anything some other way.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_float, c_int, c_int32, c_int64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libpicotron_amd.so")

PICO_BF16, PICO_F32 = 0, 1


class AttnDesc(Structure):
    """Mirror of ``pico_attn_desc``."""
    _fields_ = [
        ("B", c_int32), ("Hq", c_int32), ("Hkv", c_int32), ("Sq", c_int32), ("Sk", c_int32), ("D", c_int32),
        ("causal", c_int32), ("q_offset", c_int32), ("sm_scale", c_float), ("reserved", c_int32),
        ("q_stride", c_int64 * 3), ("k_stride", c_int64 * 3), ("v_stride", c_int64 * 3), ("o_stride", c_int64 * 3),
    ]


class RopeTables(Structure):
    """Mirror of ``pico_rope_tables``."""
    _fields_ = [("cos", c_void_p), ("sin", c_void_p), ("pitch", c_int64), ("dtype", c_int32), ("rows", c_int32)]


MAX_KV_CHUNKS = 16


class KvChunks(Structure):
    """Mirror of ``pico_kv_chunks``."""
    _fields_ = [("count", c_int32), ("chunk_len", c_int32), ("k", c_void_p * MAX_KV_CHUNKS), ("v", c_void_p * MAX_KV_CHUNKS),
                ("dk", c_void_p * MAX_KV_CHUNKS), ("dv", c_void_p * MAX_KV_CHUNKS),
                ("dk_final", c_void_p * MAX_KV_CHUNKS), ("dv_final", c_void_p * MAX_KV_CHUNKS), ("final_stride", c_int64 * 3),
                ("accumulate_mask", ctypes.c_uint32), ("reserved", ctypes.c_uint32)]


_P = c_void_p
_I64 = c_int64
SIGNATURES = {
    "pico_version": (c_char_p, []),
    "pico_last_error": (c_char_p, []),
    "pico_rmsnorm_fwd": (c_int, [_P, _P, _P, _P, _P, _P, _I64, _I64, c_float, c_int, c_int, _P]),
    "pico_rmsnorm_bwd_workspace_bytes": (_I64, [_I64, _I64]),
    "pico_rmsnorm_bwd": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int, _P, _I64, _I64, _I64, c_int, _P]),
    "pico_rmsnorm_bwd_static_max_bytes": (_I64, []),
    "pico_rmsnorm_bwd_static": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int, _I64, _I64, c_int, _P]),
    "pico_rope": (c_int, [_P, _P, _P, _P] + [_I64] * 4 + [_I64] * 6 + [_I64, _I64, c_int, c_int, c_int, _P]),
    "pico_swiglu_fwd": (c_int, [_P, _P, _P] + [_I64] * 5 + [c_int, _P]),
    "pico_swiglu_bwd": (c_int, [_P] * 5 + [_I64] * 7 + [c_int, _P]),
    "pico_lse_merge": (c_int, [_P, _P, _P, _P, _I64, _I64, c_int, _P]),
    "pico_attn_fwd": (c_int, [POINTER(AttnDesc), _P, _P, _P, _P, _P, c_int, c_int, _P]),
    "pico_attn_fwd_rope": (c_int, [POINTER(AttnDesc), _P, _P, _P, _P, _P, c_int, c_int, POINTER(RopeTables), c_int, _P, POINTER(c_int64), _P]),
    "pico_attn_bwd_rope": (c_int, [POINTER(AttnDesc)] + [_P] * 5 + [_P, _P] + [_P, POINTER(c_int64), c_int, c_int, _P, _P, POINTER(c_int64), c_int, c_int,
                                   POINTER(RopeTables), c_int, c_int, _P]),
    "pico_attn_fwd_chunks": (c_int, [POINTER(AttnDesc), _P, POINTER(KvChunks), _P, _P, c_int, c_int, POINTER(RopeTables), c_int, _P,
                                     POINTER(c_int64), _P]),
    "pico_attn_bwd_chunks": (c_int, [POINTER(AttnDesc), _P, POINTER(KvChunks), _P, _P, c_int, _P, _P, _P, POINTER(c_int64), c_int, c_int,
                                     POINTER(c_int64), c_int, POINTER(RopeTables), c_int, c_int, _P]),
    "pico_attn_bwd_preprocess": (c_int, [POINTER(AttnDesc), _P, _P, c_int, _P, _P, _P]),
    "pico_attn_bwd": (c_int, [POINTER(AttnDesc)] + [_P] * 6 + [_P, POINTER(c_int64), c_int, c_int, _P, _P, POINTER(c_int64), c_int, c_int, _P]),
    "pico_attn_bwd_fused": (c_int, [POINTER(AttnDesc)] + [_P] * 5 + [c_int, _P, _P] + [_P, POINTER(c_int64), c_int, c_int, _P, _P, POINTER(c_int64), c_int, c_int, _P]),
    "pico_cross_entropy_fwd": (c_int, [_P, _P, _P, _P, _I64, _I64, _I64, _I64, c_int, _P]),
    "pico_cross_entropy_bwd": (c_int, [_P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, c_int, _P]),
    "pico_adamw": (c_int, [_P, _P, _P, c_int, _P, _P, _I64] + [ctypes.c_float] * 5 + [_I64, ctypes.c_float, _P]),
    "pico_adamw_lp": (c_int, [_P, _P, c_int, _P, _P, _I64, c_int, c_int] + [ctypes.c_float] * 5 + [_I64, ctypes.c_float, _P]),
    "pico_adamw_multi": (c_int, [c_int, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int] + [ctypes.c_float] * 5 + [_I64, ctypes.c_float, _P]),
    "pico_convert_f32": (c_int, [_P, _P] + [_I64] * 7 + [c_int, _P]),
}

_lib = None


def lib() -> ctypes.CDLL:
    """The loaded library; raises if it was never built (no fallback path exists)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build the HIP kernels first with `python -m picotron_amd.build` "
                "(picotron_amd has no CPU or torch fallback)")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(rc: int) -> None:
    """Turn a negative pico_status into the RuntimeError the reference's Python would raise."""
    if rc != 0:
        raise RuntimeError(f"picotron_amd error {rc}: {lib().pico_last_error().decode()}")
