"""The entry point that allocates nothing (``s3r_compressed_attn_topk_static``, score buffer built into the
library) against ``s3r_compressed_attn_topk`` with a caller-provided score buffer: same kernels, so the attention
output, the log-sum-exp and the indices must agree bit for bit.  Two calls in a row, the second on a smaller input
(the shared buffer still holds the first call's scores), through the C ABI."""
import ctypes

import pytest
import torch

from speed3r_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
CODE = {torch.float32: _lib.S3R_F32, torch.bfloat16: _lib.S3R_BF16, torch.float16: _lib.S3R_F16}


def _inputs(b, h, lq, lk, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn((b, h, n, 64), generator=g).mul(0.5).to(dtype).to(DEV) for n in (lq, lk, lk))
    return q, k, v


def _call(static, q, k, v, topk, check_mem=True):
    b, h, lq, d = q.shape
    lk = k.shape[2]
    o = torch.full_like(q, float("nan"))
    lse = torch.full((b, h, lq), float("nan"), dtype=torch.float32, device=DEV)
    idx = torch.full((b, h, lq, topk), -7, dtype=torch.int32, device=DEV)
    st = lambda t: (t.stride(0), t.stride(1), t.stride(2))
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    L = _lib.lib()
    if static:
        free_before = torch.cuda.mem_get_info()[0]
        rc = L.s3r_compressed_attn_topk_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(),
                                               idx.data_ptr(), b, h, lq, lk, d, topk, *st(q), *st(k), *st(v), *st(o),
                                               0.125, CODE[q.dtype], stream)
        _lib.check(rc, "s3r_compressed_attn_topk_static")
        torch.cuda.synchronize()
        if check_mem:                                               # (the library's first launch loads its code object)
            assert torch.cuda.mem_get_info()[0] >= free_before      # the call took no device memory
    else:
        scores = torch.empty((b, h, lq, lk), dtype=torch.float32, device=DEV)
        rc = L.s3r_compressed_attn_topk(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(),
                                        idx.data_ptr(), scores.data_ptr(), b, h, lq, lk, d, topk, *st(q), *st(k), *st(v),
                                        *st(o), 0.125, CODE[q.dtype], stream)
        _lib.check(rc, "s3r_compressed_attn_topk")
        torch.cuda.synchronize()
    return o, lse, idx


@pytest.mark.parametrize("dtype,topk", [(torch.bfloat16, 64), (torch.float32, 16), (torch.float16, 8)])
def test_static_score_buffer_gives_the_same_bits_on_two_calls_the_second_smaller(dtype, topk):
    _call(True, *_inputs(1, 1, 64, 64, 99, dtype), topk, check_mem=False)      # first call on the device: symbol lookup
    for shape, seed in (((2, 3, 333, 333), 1), ((1, 2, 130, 97), 2)):
        q, k, v = _inputs(*shape, seed, dtype)
        want = _call(False, q, k, v, topk)
        got = _call(True, q, k, v, topk)
        for g, w, name in zip(got, want, ("o", "lse", "idx")):
            assert torch.equal(g, w), (name, shape)
        assert not torch.isnan(got[0].float()).any() and (got[2] >= 0).all() and (got[2] < shape[3]).all()


def test_static_score_buffer_rejects_what_does_not_fit():
    one = ctypes.c_void_p(256)
    L = _lib.lib()
    rc = L.s3r_compressed_attn_topk_static(one, one, one, one, None, one, 1, 16, 2048, 2048, 64, 16, *([64] * 12), 0.125,
                                           _lib.S3R_BF16, None)       # 64 Mi scores > 24 Mi
    assert rc == _lib.S3R_ERR_UNSUPPORTED and b"exceed" in L.s3r_last_error()
    rc = L.s3r_compressed_attn_topk_static(one, one, one, None, None, one, 1, 1, 64, 64, 64, 16, *([64] * 12), 0.125,
                                           _lib.S3R_BF16, None)
    assert rc == _lib.S3R_ERR_BAD_ARG
