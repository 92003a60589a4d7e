"""ctypes binding of the C-ABI library (include/speed3r_hip.h).

The library is the only implementation of the operators: if it is missing or fails to load,
every operator raises.  There is no fallback path.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int32, c_int64, c_void_p, POINTER
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "csrc" / "libspeed3r_hip.so"

S3R_F32, S3R_BF16, S3R_F16 = 0, 1, 2
S3R_OK = 0
S3R_ERR_BAD_ARG, S3R_ERR_UNSUPPORTED, S3R_ERR_HIP = -1, -2, -3

# name -> (restype, argtypes); mirrors include/speed3r_hip.h declaration by declaration
_i64x3 = [c_int64, c_int64, c_int64]
SIGNATURES = {
    "s3r_version": (c_char_p, []),
    "s3r_last_error": (c_char_p, []),
    "s3r_capabilities": (c_int, []),
    "s3r_pool_mean": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int64, c_int, c_int, *_i64x3, *_i64x3, c_int, c_void_p]),
    "s3r_compressed_attn_topk": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                         c_int, c_int, c_int, c_int, c_int, c_int,
                                         *_i64x3, *_i64x3, *_i64x3, *_i64x3, c_float, c_int, c_void_p]),
    "s3r_compressed_attn_topk_causal": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                         c_int, c_int, c_int, c_int, c_int, c_int,
                                         *_i64x3, *_i64x3, *_i64x3, *_i64x3, c_float, c_int, c_void_p]),
    "s3r_compressed_attn_topk_static": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                                c_int, c_int, c_int, c_int, c_int, c_int,
                                                *_i64x3, *_i64x3, *_i64x3, *_i64x3, c_float, c_int, c_void_p]),
    "s3r_topk_rows": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int64, c_int, c_void_p]),
    "s3r_select_attn": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                c_int, c_int, c_int64, c_int, c_int, c_int,
                                *_i64x3, *_i64x3, *_i64x3, *_i64x3, *_i64x3, c_float, c_int, c_void_p]),
    "s3r_select_attn_merge": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_int, c_int, c_int64, c_int, c_int, c_int,
                                      *_i64x3, *_i64x3, *_i64x3, *_i64x3, *_i64x3, *_i64x3, c_float, c_int, c_void_p]),
    "s3r_norm_rope": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_float,
                              c_int, c_int, c_int64, c_int, *_i64x3, c_int64, c_int64, c_int, c_void_p]),
    "s3r_qkv_prepass": (c_int, [c_void_p] * 8 + [c_void_p, c_void_p, c_void_p, c_int] + [c_void_p] * 4 + [c_float, c_int, c_int, c_int64,
                                c_int, c_int, *_i64x3, c_int64, c_int64, c_int, c_void_p]),
    "s3r_layer_norm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_int64, c_int, c_int64, c_int64, c_int, c_void_p]),
    "s3r_gated_merge": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int64, c_int, c_int,
                                *_i64x3, *_i64x3, *_i64x3, c_int, c_void_p]),
    "s3r_attn_bwd_delta": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int64, c_int, *_i64x3, *_i64x3,
                                   c_int, c_void_p]),
    "s3r_key_block_lists": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int64, c_int, c_int64, *_i64x3, c_int64, c_void_p]),
    "s3r_attn_bwd": (c_int, [c_void_p] * 6 + [c_void_p, c_void_p, c_void_p, c_int64] + [c_void_p] * 3
                     + [c_int, c_int, c_int64, c_int64, c_int, c_int, c_int]
                     + _i64x3 * 8 + [c_float, c_int, c_void_p]),
}

_lib = None


class Speed3rHipError(RuntimeError):
    """A C-ABI call returned a negative status."""


def lib() -> ctypes.CDLL:
    """Load (once) and return the library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} not found: the HIP library is not built. Run `python -m speed3r_amd.build` "
                "(needs hipcc). There is no non-HIP implementation of these operators.")
        handle = ctypes.CDLL(str(LIB_PATH))
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError if the library lacks a declared symbol
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


S3R_CAP_FUSED_TOPK = 1


def lib_has_fused_topk() -> bool:
    return bool(lib().s3r_capabilities() & S3R_CAP_FUSED_TOPK)


def check(rc: int, what: str) -> None:
    if rc != S3R_OK:
        msg = lib().s3r_last_error().decode("utf-8", "replace")
        raise Speed3rHipError(f"{what} failed (code {rc}): {msg}")
