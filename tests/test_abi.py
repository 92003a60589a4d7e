"""The C-ABI library loads, exports every symbol the header declares, and validates arguments
on the host before touching the device (no compute calls here)."""
import ctypes
import re
from pathlib import Path

import pytest
import torch

from speed3r_amd import _lib

ROOT = Path(__file__).resolve().parent.parent
HEADER = (ROOT / "include" / "speed3r_hip.h").read_text()
DECLARED = sorted(set(re.findall(r"\b(s3r_[a-z0-9_]+)\s*\(", HEADER)))


def test_header_declares_the_expected_entry_points():
    assert {"s3r_pool_mean", "s3r_compressed_attn_topk", "s3r_topk_rows", "s3r_select_attn", "s3r_gated_merge",
            "s3r_version", "s3r_last_error", "s3r_capabilities"} <= set(DECLARED)


@pytest.mark.parametrize("name", DECLARED)
def test_library_exports_symbol(name):
    handle = ctypes.CDLL(str(_lib.LIB_PATH))
    assert hasattr(handle, name)


def test_binding_table_covers_header():
    assert sorted(_lib.SIGNATURES) == DECLARED


def test_version_string():
    assert _lib.lib().s3r_version().decode().startswith("speed3r_hip")


def test_host_side_validation_returns_error_codes():
    L = _lib.lib()
    assert L.s3r_pool_mean(None, None, 1, 1, 64, 64, 64, 0, 0, 0, 0, 0, 0, _lib.S3R_BF16, None) == -1
    assert b"null" in L.s3r_last_error()
    assert L.s3r_topk_rows(None, None, 1, 1, 1, 4, None) == -1
    assert L.s3r_topk_rows(ctypes.c_void_p(16), ctypes.c_void_p(16), 1, 8, 8, 65, None) == -2      # K > 64
    assert L.s3r_select_attn(ctypes.c_void_p(16), ctypes.c_void_p(16), ctypes.c_void_p(16), ctypes.c_void_p(16),
                             ctypes.c_void_p(16), None, 1, 1, 64, 128, 64, 4, *([0] * 15), 0.125, _lib.S3R_BF16,
                             None) == -2                                                            # head_dim > 64
    assert b"head_dim" in L.s3r_last_error()
    assert L.s3r_compressed_attn_topk(ctypes.c_void_p(16), ctypes.c_void_p(16), ctypes.c_void_p(16), ctypes.c_void_p(16),
                                      None, ctypes.c_void_p(16), None, 1, 1, 8, 8, 64, 12, *([0] * 12), 0.125,
                                      _lib.S3R_BF16, None) == -2                                    # K not a power of two
    assert L.s3r_gated_merge(ctypes.c_void_p(16), ctypes.c_void_p(16), ctypes.c_void_p(16), ctypes.c_void_p(16),
                             1, 1, 64, 64, 64, *([0] * 9), 7, None) == -2                           # unknown dtype
    one = ctypes.c_void_p(16)

    def causal(o=one, idx=one, scores=one, k=8, d=64):
        return L.s3r_compressed_attn_topk_causal(one, one, one, o, None, idx, scores, 1, 1, 8, 8, d, k, *([0] * 12),
                                                 0.125, _lib.S3R_BF16, None)

    assert causal(o=None) == _lib.S3R_ERR_BAD_ARG                    # the causal entry always writes o
    assert causal(scores=None) == _lib.S3R_ERR_BAD_ARG               # its indices are selected from the score buffer
    assert b"score buffer" in L.s3r_last_error()
    assert causal(k=12) == _lib.S3R_ERR_UNSUPPORTED and causal(d=128) == _lib.S3R_ERR_UNSUPPORTED


def test_backward_entry_points_validate_on_the_host():
    L = _lib.lib()
    z3 = (0, 0, 0)
    assert L.s3r_attn_bwd_delta(None, None, None, 1, 1, 64, 64, *z3, *z3, _lib.S3R_BF16, None) == _lib.S3R_ERR_BAD_ARG
    one = ctypes.c_void_p(16)      # any non-null, 16-byte aligned address: validation never dereferences it
    st = (64 * 64, 64 * 64, 64)

    def bwd(dq=one, dk=one, dv=one, idx=None, lists=None, off=None, d=64, block=64, dtype=_lib.S3R_BF16, scale=0.125, q_st=st):
        return L.s3r_attn_bwd(one, one, one, one, one, one, idx, lists, off, 0, dq, dk, dv, 1, 1, 64, 64, d, block, 4,
                              *q_st, *st, *st, *st, *st, *st, *st, *z3, scale, dtype, None)

    assert bwd(dq=None, dk=None, dv=None) == _lib.S3R_ERR_BAD_ARG           # no gradient requested
    assert bwd(dk=None) == _lib.S3R_ERR_BAD_ARG                             # dk and dv come together
    assert bwd(idx=one) == _lib.S3R_ERR_BAD_ARG                             # selection dk/dv without the key-centric lists
    assert bwd(d=32) == _lib.S3R_ERR_UNSUPPORTED
    assert bwd(idx=one, lists=one, off=one, block=32) == _lib.S3R_ERR_UNSUPPORTED   # selection blocks of 64 or 16 tokens
    assert bwd(dtype=_lib.S3R_F32) == _lib.S3R_ERR_UNSUPPORTED and bwd(scale=0.0) == _lib.S3R_ERR_UNSUPPORTED
    assert bwd(q_st=(64 * 64, 64 * 64, 1 << 20)) == _lib.S3R_ERR_UNSUPPORTED  # row stride beyond the 32-bit tile offsets
    assert bwd(q_st=(64 * 64, 64 * 64, 60)) == _lib.S3R_ERR_BAD_ARG          # rows not 16-byte aligned
    assert b"s3r_attn_bwd" in L.s3r_last_error()
    assert L.s3r_layer_norm(None, one, one, None, 1e-6, 1, 64, 64, 64, _lib.S3R_BF16, None) == _lib.S3R_ERR_BAD_ARG
    assert L.s3r_layer_norm(one, one, one, None, 1e-6, 1, 12, 64, 64, _lib.S3R_BF16, None) == _lib.S3R_ERR_UNSUPPORTED
    assert b"s3r_layer_norm" in L.s3r_last_error()
    assert L.s3r_key_block_lists(None, one, one, 1, 1, 4, 4, 4, *z3, 16, None) == _lib.S3R_ERR_BAD_ARG
    assert L.s3r_key_block_lists(one, one, one, 1, 1, 4, 4, 4, *z3, 15, None) == _lib.S3R_ERR_BAD_ARG      # list_stride < nqb * K
    assert L.s3r_key_block_lists(one, one, one, 1, 1, 1 << 30, 4, 4, *z3, 1 << 32, None) == _lib.S3R_ERR_UNSUPPORTED
    assert b"s3r_key_block_lists" in L.s3r_last_error()


def test_operators_refuse_cpu_tensors():
    import speed3r_amd as s3r

    x = torch.zeros((1, 1, 64, 64), dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="HIP device"):
        s3r.pool_mean(x, 64)
    with pytest.raises(RuntimeError, match="HIP device"):
        s3r.topk_blocksparse_attention(x, x, x, torch.zeros((1, 1, 1, 1), dtype=torch.int32), 64)


def test_reference_signature_asserts():
    import speed3r_amd as s3r

    x = torch.zeros((1, 1, 64, 64), dtype=torch.bfloat16)
    with pytest.raises(AssertionError):
        s3r.flash_attn_topk_func(x, x, x, 128)                      # K > BLOCK_N
    with pytest.raises(AssertionError):
        s3r.topk_blocksparse_attention(x, x, x, torch.zeros((1, 1, 1, 1), dtype=torch.int64), 64)   # idx dtype
    with pytest.raises(AssertionError):
        s3r.topk_blocksparse_attention(x, x, x, torch.zeros((1, 1, 1, 1), dtype=torch.int32), 48)   # block size
