"""Torch-facing wrappers of the C-ABI entry points.

PyTorch supplies device memory and the current HIP stream; the arithmetic is done by the
hand-written gfx950 kernels behind ``include/speed3r_hip.h``.  Every function takes and
returns HIP-device tensors and raises if the library is not built -- there is no CPU or
eager fallback.

Layouts follow the reference operators: q/k/v/o are ``[B, H, L, D]`` with a contiguous last
dimension; indices are int32 ``[B, H, n_query_blocks, K]`` in block units.
"""
from __future__ import annotations

import math
import os
from typing import Optional, Tuple

import torch

from .. import _lib


_DTYPE_CODE = {torch.float32: _lib.S3R_F32, torch.bfloat16: _lib.S3R_BF16, torch.float16: _lib.S3R_F16}


def _code(t: torch.Tensor) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {t.dtype}; expected float32, bfloat16 or float16") from None


def _need_device(*ts: torch.Tensor) -> None:
    for t in ts:
        if not t.is_cuda:
            raise RuntimeError("speed3r_amd operators run on HIP device tensors only (got a CPU tensor)")


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _last_contig(t: torch.Tensor) -> torch.Tensor:
    return t if t.stride(-1) == 1 else t.contiguous()


def _forward_only(*ts: torch.Tensor) -> None:
    if torch.is_grad_enabled() and any(t.requires_grad for t in ts):
        raise RuntimeError("speed3r_amd operators are forward-only; call them under torch.no_grad()")


def pool_mean(x: torch.Tensor, block: int) -> torch.Tensor:
    """Mean over non-overlapping runs of ``block`` tokens: [B,H,N,D] -> [B,H,ceil(N/block),D].

    ``x`` may be any strided view with a contiguous last dimension (e.g. a head-major view of
    the packed qkv projection).  A ragged tail block is a mean over its valid tokens.
    """
    _need_device(x)
    _forward_only(x)
    x = _last_contig(x)
    b, h, n, d = x.shape
    nc = -(-n // block)
    y = torch.empty((b, h, nc, d), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        rc = _lib.lib().s3r_pool_mean(x.data_ptr(), y.data_ptr(), b, h, n, d, block,
                                      x.stride(0), x.stride(1), x.stride(2),
                                      y.stride(0), y.stride(1), y.stride(2), _code(x), _stream(x))
    _lib.check(rc, "s3r_pool_mean")
    return y


def pool_qkv_packed(qkv: torch.Tensor, num_heads: int, block: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Pool the packed projection ``[B, N, 3*H*D]`` (layout ``(qkv h d)``) in one launch.

    Returns pooled q, k, v as ``[B, H, Nc, D]`` views of one ``[B, 3H, Nc, D]`` buffer.
    """
    b, n, c3 = qkv.shape
    d = c3 // (3 * num_heads)
    view = qkv.view(b, n, 3 * num_heads, d).permute(0, 2, 1, 3)  # [B, 3H, N, D], strided
    y = pool_mean(view, block)
    return y[:, :num_heads], y[:, num_heads:2 * num_heads], y[:, 2 * num_heads:]


# largest fp32 score buffer compressed_attn_topk allocates for its own use (a caller that asks for the scores gets them whole)
SCORE_BUFFER_BYTES = 1 << 30
CAUSAL_SCORE_BYTES = 8 << 30   # the causal variant's score buffer is not banded


def compressed_attn_topk(q: torch.Tensor, k: torch.Tensor, v: Optional[torch.Tensor], topk: Optional[int],
                         softmax_scale: Optional[float] = None, return_scores: bool = False,
                         return_lse: bool = False, materialize_scores: Optional[bool] = None,
                         out: Optional[torch.Tensor] = None, causal: bool = False):
    """Dense attention over pooled tokens plus, if ``topk`` is given, the top-k columns of the
    raw scores per query row.

    Returns ``(o, idx)`` with optional ``scores`` ([B,H,Lq,Lk] fp32) and ``lse`` appended when
    requested.  ``materialize_scores`` forces (True) or forbids (False) the fp32 score buffer.  By
    default the selection is fused into the attention kernel wherever the library has it (bf16/fp16,
    head_dim 64, top-k a power of two up to 32): the scores never leave the chip.  Otherwise the scores
    go through HBM (attention kernel, then the row-wise top-k kernel).

    ``v=None`` asks for the indices alone (``o`` is returned as ``None``; fused selection only): the
    attention output and the indices come from two different kernels, and a caller with two streams runs
    them side by side, see :func:`sparse_global_attention`.

    ``out``: a ``[B,H,Lq,D]`` tensor (or view, any strides on the first three dimensions, e.g. the
    ``permute(0, 2, 1, 3)`` of a ``[B,Lq,H,D]`` buffer) that receives the attention output instead of a fresh one.

    ``causal``: the reference kernel's IS_CAUSAL variant (flash_attention_topk.py:71,93), never taken by the reference
    layer: query i attends the keys j <= i and ranks the keys below ``min((i // 64 + 1) * 64, Lk)``, those above i
    with the score -inf.  Generic kernels with a full ``[B,H,Lq,Lk]`` fp32 score buffer (at most
    ``CAUSAL_SCORE_BYTES``); with ``return_scores`` the columns a row does not rank are returned as NaN.
    """
    if causal:
        assert v is not None and out is None, "causal: attention output and indices come from one call, into a fresh tensor"
        _need_device(q, k, v)
        _forward_only(q, k, v)
        q, k, v = (_last_contig(t) for t in (q, k, v))
        assert q.dtype == k.dtype == v.dtype, "q, k, v must share a dtype"
        b, h, lq, d = q.shape
        lk = k.shape[2]
        assert k.shape == (b, h, lk, d) and v.shape == (b, h, lk, d), "k/v shape mismatch"
        scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(d)
        o = torch.empty_like(q, memory_format=torch.contiguous_format)
        idx = torch.empty((b, h, lq, topk), dtype=torch.int32, device=q.device) if topk else None
        lse = torch.empty((b, h, lq), dtype=torch.float32, device=q.device) if return_lse else None
        scores = None
        if topk or return_scores:
            if 4 * b * h * lq * lk > CAUSAL_SCORE_BYTES:
                raise RuntimeError(f"causal top-k keeps all {b}x{h}x{lq}x{lk} fp32 scores in one buffer; that exceeds "
                                   f"CAUSAL_SCORE_BYTES = {CAUSAL_SCORE_BYTES}")
            scores = torch.full((b, h, lq, lk), float("nan"), dtype=torch.float32, device=q.device) if return_scores \
                else torch.empty((b, h, lq, lk), dtype=torch.float32, device=q.device)
        st3 = lambda t: (t.stride(0), t.stride(1), t.stride(2))
        with torch.cuda.device(q.device):
            rc = _lib.lib().s3r_compressed_attn_topk_causal(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr() if lse is not None else None,
                idx.data_ptr() if idx is not None else None, scores.data_ptr() if scores is not None else None,
                b, h, lq, lk, d, topk or 0, *st3(q), *st3(k), *st3(v), *st3(o), scale, _code(q), _stream(q))
        _lib.check(rc, "s3r_compressed_attn_topk_causal")
        res = [o, idx]
        if return_scores:
            res.append(scores)
        if return_lse:
            res.append(lse)
        return tuple(res)
    indices_only = v is None
    if indices_only:
        assert topk and not return_scores and not return_lse and materialize_scores is not True, \
            "v=None (indices only) needs top-k without a score buffer"
        v = k
        materialize_scores = False
    _need_device(q, k, v)
    _forward_only(q, k, v)
    q, k, v = (_last_contig(t) for t in (q, k, v))
    assert q.dtype == k.dtype == v.dtype, "q, k, v must share a dtype"
    b, h, lq, d = q.shape
    lk = k.shape[2]
    assert k.shape == (b, h, lk, d) and v.shape == (b, h, lk, d), "k/v shape mismatch"
    scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(d)
    if out is not None:
        assert not indices_only and out.shape == q.shape and out.dtype == q.dtype and out.device == q.device \
            and out.stride(-1) == 1, "out must be a [B,H,Lq,D] tensor of q's dtype and device, last dimension contiguous"
    o = None if indices_only else out if out is not None else torch.empty_like(q, memory_format=torch.contiguous_format)
    idx = torch.empty((b, h, lq, topk), dtype=torch.int32, device=q.device) if topk else None
    fused_ok = (q.dtype != torch.float32 and d == 64 and topk in (1, 2, 4, 8, 16, 32) and lk <= (1 << 21)
                and _lib.lib_has_fused_topk())
    want_scores = return_scores or (materialize_scores is True) or (
        bool(topk) and materialize_scores is None and not fused_ok)
    if materialize_scores is False and topk and not fused_ok:
        raise RuntimeError("fused top-k is not available for this dtype/shape; allow a score buffer")
    lse = torch.empty((b, h, lq), dtype=torch.float32, device=q.device) if return_lse else None
    st3 = lambda t: (t.stride(0), t.stride(1), t.stride(2))

    def launch(q_, o_, lse_, idx_, scores_, rows):
        with torch.cuda.device(q.device):
            rc = _lib.lib().s3r_compressed_attn_topk(
                q_.data_ptr(), k.data_ptr(), None if indices_only else v.data_ptr(), None if indices_only else o_.data_ptr(),
                lse_.data_ptr() if lse_ is not None else None,
                idx_.data_ptr() if idx_ is not None else None,
                scores_.data_ptr() if scores_ is not None else None,
                b, h, rows, lk, d, topk or 0, *st3(q_), *st3(k), *st3(v),
                *((0, 0, 0) if indices_only else st3(o_)), scale, _code(q), _stream(q))
        _lib.check(rc, "s3r_compressed_attn_topk")

    rows_per_pass = max(128, (SCORE_BUFFER_BYTES // (4 * b * h * lk)) // 128 * 128)
    if want_scores and not return_scores and lq > rows_per_pass:
        # top-k values without a fused kernel (fp32, top-k 64, ...) on many pooled tokens: the score buffer holds a
        # band of query rows at a time instead of the whole [Lq, Lk] matrix (16.9 GB at a million tokens)
        scores = torch.empty((b, h, rows_per_pass, lk), dtype=torch.float32, device=q.device)
        for r0 in range(0, lq, rows_per_pass):
            r1 = min(lq, r0 + rows_per_pass)
            idx_c = torch.empty((b, h, r1 - r0, topk), dtype=torch.int32, device=q.device) if topk else None
            lse_c = torch.empty((b, h, r1 - r0), dtype=torch.float32, device=q.device) if return_lse else None
            launch(q[:, :, r0:r1], o[:, :, r0:r1], lse_c, idx_c, scores, r1 - r0)
            if idx_c is not None:
                idx[:, :, r0:r1] = idx_c
            if lse_c is not None:
                lse[:, :, r0:r1] = lse_c
        scores = None
    else:
        scores = torch.empty((b, h, lq, lk), dtype=torch.float32, device=q.device) if want_scores else None
        launch(q, o, lse, idx, scores, lq)
    out = [o, idx]
    if return_scores:
        out.append(scores)
    if return_lse:
        out.append(lse)
    return tuple(out)


def topk_rows(scores: torch.Tensor, k: int) -> torch.Tensor:
    """Exact top-k columns of each row of an fp32 matrix ``[..., rows, cols]`` -> int32 ``[..., rows, k]``.

    Order: descending score, equal scores lowest column first, +0.0 above -0.0; if
    ``cols < k`` the trailing slots hold ``cols - 1``.
    """
    _need_device(scores)
    assert scores.dtype == torch.float32, "scores must be float32"
    scores = scores.contiguous()
    cols = scores.shape[-1]
    rows = scores.numel() // cols
    idx = torch.empty((*scores.shape[:-1], k), dtype=torch.int32, device=scores.device)
    with torch.cuda.device(scores.device):
        rc = _lib.lib().s3r_topk_rows(scores.data_ptr(), idx.data_ptr(), rows, cols, cols, k, _stream(scores))
    _lib.check(rc, "s3r_topk_rows")
    return idx


def _as_64_token_blocks(idx: torch.Tensor, block: int, n: int) -> torch.Tensor:
    """Index lists over blocks of 128 or 256 tokens rewritten for the 64-token kernels.

    A query block of ``r * 64`` rows is ``r`` consecutive 64-row blocks with the same list, and a listed key block is
    the run of its ``r`` 64-token blocks in order, so the rewritten tensor is ``[B,H,ceil(N/64),K*r]``: the same keys
    in the same order for every query row (entries below zero stay -1; runs reaching beyond ``N`` are cut by the
    kernels' own ``start >= N`` rule)."""
    r = block // 64
    b, h, nqb, kk = idx.shape
    sub = torch.arange(r, device=idx.device, dtype=torch.int32)
    fine = torch.where(idx[..., None] >= 0, idx[..., None] * r + sub, idx.new_full((), -1))
    return fine.reshape(b, h, nqb, kk * r).repeat_interleave(r, dim=2)[:, :, :-(-n // 64)].contiguous()


def select_attn(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, idx: torch.Tensor, block: int,
                softmax_scale: Optional[float] = None, return_lse: bool = False):
    """Attention of each ``block``-row query block over the key blocks listed in ``idx``."""
    _need_device(q, k, v, idx)
    _forward_only(q, k, v)
    q, k, v, idx = (_last_contig(t) for t in (q, k, v, idx))
    assert q.dtype == k.dtype == v.dtype, "q, k, v must share a dtype"
    assert idx.dtype == torch.int32, "topk_idx must be int32"
    b, h, n, d = q.shape
    assert k.shape == q.shape and v.shape == q.shape, "q, k, v must share a shape"
    nqb = -(-n // block)
    assert idx.shape[:3] == (b, h, nqb), f"topk_idx shape {tuple(idx.shape)} does not match {(b, h, nqb, 'K')}"
    if block in (128, 256):
        idx, block = _as_64_token_blocks(idx, block, n), 64
    kk = idx.shape[3]
    scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(d)
    o = torch.empty_like(q, memory_format=torch.contiguous_format)
    lse = torch.empty((b, h, n), dtype=torch.float32, device=q.device) if return_lse else None
    with torch.cuda.device(q.device):
        rc = _lib.lib().s3r_select_attn(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), idx.data_ptr(), o.data_ptr(),
            lse.data_ptr() if lse is not None else None,
            b, h, n, d, block, kk,
            q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1), k.stride(2),
            v.stride(0), v.stride(1), v.stride(2), o.stride(0), o.stride(1), o.stride(2),
            idx.stride(0), idx.stride(1), idx.stride(2), scale, _code(q), _stream(q))
    _lib.check(rc, "s3r_select_attn")
    return (o, lse) if return_lse else o


def gated_merge(o_cmp: torch.Tensor, o_sel: torch.Tensor, gate: torch.Tensor, block: int) -> torch.Tensor:
    """``out[b,n,h*D+d] = gate[b,h,n,0]*o_cmp[b,h,n//block,d] + gate[b,h,n,1]*o_sel[b,h,n,d]`` -> [B,N,H*D].

    ``gate`` is ``[B,H,N,2]`` in any strided form with a contiguous pair (the reference's
    ``'b n (h g) -> b h n g'`` view of the gate projection qualifies).
    """
    _need_device(o_cmp, o_sel, gate)
    _forward_only(o_cmp, o_sel, gate)
    o_cmp, o_sel, gate = (_last_contig(t) for t in (o_cmp, o_sel, gate))
    assert o_cmp.dtype == o_sel.dtype == gate.dtype, "o_cmp, o_sel, gate must share a dtype"
    b, h, n, d = o_sel.shape
    nc = -(-n // block)
    assert o_cmp.shape == (b, h, nc, d), f"o_cmp shape {tuple(o_cmp.shape)} != {(b, h, nc, d)}"
    assert gate.shape == (b, h, n, 2), f"gate shape {tuple(gate.shape)} != {(b, h, n, 2)}"
    out = torch.empty((b, n, h * d), dtype=o_sel.dtype, device=o_sel.device)
    with torch.cuda.device(o_sel.device):
        rc = _lib.lib().s3r_gated_merge(
            o_cmp.data_ptr(), o_sel.data_ptr(), gate.data_ptr(), out.data_ptr(), b, h, n, d, block,
            o_cmp.stride(0), o_cmp.stride(1), o_cmp.stride(2), o_sel.stride(0), o_sel.stride(1), o_sel.stride(2),
            gate.stride(0), gate.stride(1), gate.stride(2), _code(o_sel), _stream(o_sel))
    _lib.check(rc, "s3r_gated_merge")
    return out


def norm_rope(x: torch.Tensor, positions: Optional[torch.Tensor], cos_tab: Optional[torch.Tensor],
              sin_tab: Optional[torch.Tensor], ln_weight: Optional[torch.Tensor] = None,
              ln_bias: Optional[torch.Tensor] = None, eps: float = 1e-5) -> Optional[torch.Tensor]:
    """``RoPE2D(LayerNorm(x), positions)`` for one ``[B,H,N,64]`` tensor in one pass -> contiguous ``[B,H,N,64]``.

    ``positions``: integer ``[B,N,2]`` (or None: no rotation); ``cos_tab``/``sin_tab``: ``[P,16]`` tables in x's dtype
    (``RoPE2D.tables``); ``ln_weight``/``ln_bias``: LayerNorm(64) parameters (None: no normalisation).
    Returns None when the library has no kernel for the shape (head_dim other than 64)."""
    _need_device(x)
    _forward_only(x)
    x = _last_contig(x)
    b, h, n, d = x.shape
    if d != 64:
        return None
    pos32 = None
    p = 0
    if positions is not None:
        assert positions.shape == (b, n, 2), f"positions shape {tuple(positions.shape)} != {(b, n, 2)}"
        assert cos_tab is not None and sin_tab is not None and cos_tab.shape == sin_tab.shape and cos_tab.shape[1] == 16
        assert cos_tab.dtype == x.dtype and sin_tab.dtype == x.dtype, "tables must have x's dtype"
        pos32 = positions.to(device=x.device, dtype=torch.int32).contiguous()
        cos_tab, sin_tab = cos_tab.contiguous(), sin_tab.contiguous()
        p = cos_tab.shape[0]
    w = ln_weight.detach().to(x.dtype).contiguous() if ln_weight is not None else None
    bias = ln_bias.detach().to(x.dtype).contiguous() if (ln_bias is not None and w is not None) else None
    y = torch.empty((b, h, n, d), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        rc = _lib.lib().s3r_norm_rope(
            x.data_ptr(), y.data_ptr(), pos32.data_ptr() if pos32 is not None else None,
            cos_tab.data_ptr() if pos32 is not None else None, sin_tab.data_ptr() if pos32 is not None else None, p,
            w.data_ptr() if w is not None else None, bias.data_ptr() if bias is not None else None, float(eps),
            b, h, n, d, x.stride(0), x.stride(1), x.stride(2),
            pos32.stride(0) if pos32 is not None else 0, pos32.stride(1) if pos32 is not None else 0,
            _code(x), _stream(x))
    _lib.check(rc, "s3r_norm_rope")
    return y


def qkv_prepass(qkv: torch.Tensor, num_heads: int, block: int, positions: Optional[torch.Tensor],
                cos_tab: Optional[torch.Tensor], sin_tab: Optional[torch.Tensor],
                q_ln: Optional[Tuple[torch.Tensor, Optional[torch.Tensor]]] = None,
                k_ln: Optional[Tuple[torch.Tensor, Optional[torch.Tensor]]] = None, eps: float = 1e-5):
    """The layer's pre-pass over the packed projection ``[B, N, 3*H*64]`` (layout ``(qkv h d)``) in one kernel:
    returns ``(q, k, v, q_c, k_c, v_c)`` -- q, k ``[B,H,N,64]`` contiguous after LayerNorm (``q_ln``/``k_ln`` = (weight,
    bias) or None) and RoPE2D at ``positions`` (None: no rotation), v the strided view of the projection, and the
    block means of the RAW q, k, v ``[B,H,ceil(N/block),64]``.  Same bits as :func:`pool_qkv_packed` followed by
    :func:`norm_rope` on q and k.  Returns None when the library has no kernel for the shape (head_dim other than 64)."""
    _need_device(qkv)
    _forward_only(qkv)
    b, n, c3 = qkv.shape
    d = c3 // (3 * num_heads)
    if d != 64 or c3 != 3 * num_heads * 64 or qkv.stride(-1) != 1:
        return None
    assert (q_ln is None) == (k_ln is None), "q and k are normalised together or not at all"
    h = num_heads
    q, k, v = qkv.view(b, n, 3, h, d).permute(2, 0, 3, 1, 4).unbind(0)   # each [B,H,N,D], common strides
    nc = -(-n // block)
    q_out, k_out = (torch.empty((b, h, n, d), dtype=qkv.dtype, device=qkv.device) for _ in range(2))
    qc, kc, vc = (torch.empty((b, h, nc, d), dtype=qkv.dtype, device=qkv.device) for _ in range(3))
    pos32 = None
    p = 0
    if positions is not None:
        assert positions.shape == (b, n, 2), f"positions shape {tuple(positions.shape)} != {(b, n, 2)}"
        assert cos_tab is not None and sin_tab is not None and cos_tab.shape == sin_tab.shape and cos_tab.shape[1] == 16
        assert cos_tab.dtype == qkv.dtype and sin_tab.dtype == qkv.dtype, "tables must have the tokens' dtype"
        pos32 = positions.to(device=qkv.device, dtype=torch.int32).contiguous()
        cos_tab, sin_tab = cos_tab.contiguous(), sin_tab.contiguous()
        p = cos_tab.shape[0]

    def par(t):
        return t.detach().to(qkv.dtype).contiguous() if t is not None else None

    qw, qb = (par(q_ln[0]), par(q_ln[1])) if q_ln is not None else (None, None)
    kw, kb = (par(k_ln[0]), par(k_ln[1])) if k_ln is not None else (None, None)
    ptr = lambda t: t.data_ptr() if t is not None else None
    with torch.cuda.device(qkv.device):
        rc = _lib.lib().s3r_qkv_prepass(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), q_out.data_ptr(), k_out.data_ptr(), qc.data_ptr(), kc.data_ptr(),
            vc.data_ptr(), ptr(pos32), ptr(cos_tab) if pos32 is not None else None, ptr(sin_tab) if pos32 is not None else None, p,
            ptr(qw), ptr(qb), ptr(kw), ptr(kb), float(eps), b, h, n, d, block, q.stride(0), q.stride(1), q.stride(2),
            pos32.stride(0) if pos32 is not None else 0, pos32.stride(1) if pos32 is not None else 0, _code(qkv), _stream(qkv))
    _lib.check(rc, "s3r_qkv_prepass")
    return q_out, k_out, v, qc, kc, vc


def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], eps: float) -> Optional[torch.Tensor]:
    """``F.layer_norm(x, (C,), weight, bias, eps)`` over the last dimension of token rows in one pass (inference).

    Returns None when the library has no kernel for the shape (rows that are not a multiple of 16 bytes or longer
    than 512 16-byte chunks, a tensor whose leading dimensions do not collapse to one row stride)."""
    _need_device(x)
    _forward_only(x)
    c = x.shape[-1]
    vec = 16 // x.element_size()
    if x.dtype not in (torch.bfloat16, torch.float16, torch.float32) or c % vec or c // vec > 512 or x.numel() == 0:
        return None
    x2 = x.reshape(-1, c) if x.is_contiguous() else None
    if x2 is None:
        return None
    w = weight.detach().to(x.dtype).contiguous()
    b = bias.detach().to(x.dtype).contiguous() if bias is not None else None
    y = torch.empty_like(x2)
    with torch.cuda.device(x.device):
        rc = _lib.lib().s3r_layer_norm(x2.data_ptr(), y.data_ptr(), w.data_ptr(), b.data_ptr() if b is not None else None,
                                       float(eps), x2.shape[0], c, x2.stride(0), y.stride(0), _code(x), _stream(x))
    _lib.check(rc, "s3r_layer_norm")
    return y.view(x.shape)


def select_attn_merge(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, idx: torch.Tensor, o_cmp: torch.Tensor,
                      gate: torch.Tensor, block: int, softmax_scale: Optional[float] = None) -> Optional[torch.Tensor]:
    """``select_attn`` with ``gated_merge`` in its epilogue -> ``[B,N,H*D]``; bit-identical to the two calls, without the
    round trip of the selection output through memory.  Returns ``None`` when the library has no fused kernel for the
    shape (the caller then runs the two operators)."""
    _need_device(q, k, v, idx, o_cmp, gate)
    _forward_only(q, k, v, o_cmp, gate)
    q, k, v, idx, o_cmp, gate = (_last_contig(t) for t in (q, k, v, idx, o_cmp, gate))
    assert q.dtype == k.dtype == v.dtype == o_cmp.dtype == gate.dtype, "q, k, v, o_cmp, gate must share a dtype"
    assert idx.dtype == torch.int32, "topk_idx must be int32"
    b, h, n, d = q.shape
    assert k.shape == q.shape and v.shape == q.shape, "q, k, v must share a shape"
    nqb = -(-n // block)
    assert idx.shape[:3] == (b, h, nqb), f"topk_idx shape {tuple(idx.shape)} does not match {(b, h, nqb, 'K')}"
    assert o_cmp.shape == (b, h, nqb, d), f"o_cmp shape {tuple(o_cmp.shape)} != {(b, h, nqb, d)}"
    assert gate.shape == (b, h, n, 2), f"gate shape {tuple(gate.shape)} != {(b, h, n, 2)}"
    if block in (128, 256):  # 64-row query blocks share their parent's list and its row of the compressed output
        o_cmp = o_cmp.repeat_interleave(block // 64, dim=2)[:, :, :-(-n // 64)].contiguous()
        idx, block = _as_64_token_blocks(idx, block, n), 64
    if q.dtype == torch.float32 or d != 64 or block not in (64, 16) or idx.shape[3] > 64:
        return None
    scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(d)
    out = torch.empty((b, n, h * d), dtype=q.dtype, device=q.device)
    with torch.cuda.device(q.device):
        rc = _lib.lib().s3r_select_attn_merge(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), idx.data_ptr(), o_cmp.data_ptr(), gate.data_ptr(), out.data_ptr(),
            b, h, n, d, block, idx.shape[3],
            q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1), k.stride(2),
            v.stride(0), v.stride(1), v.stride(2), idx.stride(0), idx.stride(1), idx.stride(2),
            o_cmp.stride(0), o_cmp.stride(1), o_cmp.stride(2), gate.stride(0), gate.stride(1), gate.stride(2),
            scale, _code(q), _stream(q))
    if rc == _lib.S3R_ERR_UNSUPPORTED:
        return None
    _lib.check(rc, "s3r_select_attn_merge")
    return out


# ---- backward of the two attention operators --------------------------------------------------------------------

def bwd_supported(q: torch.Tensor, block: int = 64) -> bool:
    """The backward kernels are built for bf16/fp16, head_dim 64, blocks of 64 or 16 tokens."""
    return q.dtype in (torch.bfloat16, torch.float16) and q.shape[-1] == 64 and block in (64, 16)


def key_block_lists(idx: torch.Tensor, n_key_blocks: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Key-centric view of the index tensor ``[B,H,Nq_blocks,K]``: for every (b, h) the query-block ids grouped by
    the key block they list, one entry per occurrence, ascending within a group, ``[B,H,Nq_blocks*K]`` int32, and the
    group offsets ``[B,H,n_key_blocks+1]``; entries < 0 or >= n_key_blocks appear in no group (the tail of the list
    tensor behind the last offset is then unspecified).  The reference's count + stable argsort + reorder
    (topk_blocksparse_attention.py:423-554)."""
    _need_device(idx)
    assert idx.dtype == torch.int32 and idx.dim() == 4 and n_key_blocks > 0
    idx = _last_contig(idx)
    b, h, nqb, kk = idx.shape
    lists = torch.empty((b, h, nqb * kk), dtype=torch.int32, device=idx.device)
    off = torch.empty((b, h, n_key_blocks + 1), dtype=torch.int32, device=idx.device)
    with torch.cuda.device(idx.device):
        rc = _lib.lib().s3r_key_block_lists(idx.data_ptr(), lists.data_ptr(), off.data_ptr(), b, h, nqb, kk, n_key_blocks,
                                            idx.stride(0), idx.stride(1), idx.stride(2), nqb * kk, _stream(idx))
    _lib.check(rc, "s3r_key_block_lists")
    return lists, off


def key_lists_ascending(lists: torch.Tensor, offs: torch.Tensor) -> bool:
    """Whether every group of ``lists`` ([B,H,L] int32, groups delimited by ``offs`` [B,H,n_key_blocks+1]) is ascending,
    as :func:`key_block_lists` builds them.  The dK/dV kernel for 16-token blocks merges the lists of four neighbouring
    key blocks and relies on that order: on a list that is not ascending it skips entries and the gradients come out
    incomplete WITHOUT an error.  Works on CPU and GPU tensors (on the GPU: a few small kernels and one
    synchronisation)."""
    b, h, length = lists.shape
    if length < 2:
        return True
    dev = lists.device
    starts = torch.zeros((b, h, length + 1), dtype=torch.bool, device=dev)
    starts.scatter_(2, offs.long().clamp(0, length), True)                      # a pair that straddles a group start is free
    second = torch.arange(1, length, device=dev)
    beyond = second >= offs[..., -1:].long()                                     # so is the unspecified tail
    ok = (lists[..., 1:] >= lists[..., :-1]) | starts[..., 1:length] | beyond
    return bool(ok.all())


def attn_bwd_delta(o: torch.Tensor, dout: torch.Tensor) -> torch.Tensor:
    """``delta[b,h,n] = sum_d o * dout`` in fp32."""
    _need_device(o, dout)
    o, dout = _last_contig(o), _last_contig(dout)
    b, h, n, d = o.shape
    delta = torch.empty((b, h, n), dtype=torch.float32, device=o.device)
    with torch.cuda.device(o.device):
        rc = _lib.lib().s3r_attn_bwd_delta(o.data_ptr(), dout.data_ptr(), delta.data_ptr(), b, h, n, d,
                                           o.stride(0), o.stride(1), o.stride(2),
                                           dout.stride(0), dout.stride(1), dout.stride(2), _code(o), _stream(o))
    _lib.check(rc, "s3r_attn_bwd_delta")
    return delta


def attn_bwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, o: torch.Tensor, dout: torch.Tensor, lse: torch.Tensor,
             idx: Optional[torch.Tensor] = None, block: int = 64, softmax_scale: Optional[float] = None,
             need_dq: bool = True, need_dkv: bool = True, delta: Optional[torch.Tensor] = None,
             key_lists: Optional[Tuple[torch.Tensor, torch.Tensor]] = None, check_lists: Optional[bool] = None):
    """Gradients ``(dq, dk, dv)`` of an attention forward with output ``o`` and log-sum-exp ``lse``:
    selection attention over the blocks of ``idx`` ([B,H,Nq_blocks,K] int32), or dense attention (``idx=None``).
    ``delta`` (:func:`attn_bwd_delta`) and ``key_lists`` (:func:`key_block_lists`) are computed here unless given.
    Caller-built ``key_lists`` must be ascending within every group (see :func:`key_lists_ascending`: with 16-token
    blocks anything else gives silently incomplete dk, dv); ``check_lists=True`` (default: the environment variable
    ``S3R_CHECK_LISTS=1``) verifies that here, at the price of a device synchronisation."""
    _need_device(q, k, v, o, dout, lse)
    assert bwd_supported(q, block), "attention backward: built for bf16/fp16, head_dim 64, block 64 or 16"
    q, k, v, o, dout = (_last_contig(t) for t in (q, k, v, o, dout))
    lse = lse.contiguous()
    b, h, lq, d = q.shape
    lk = k.shape[2]
    scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(d)
    if delta is None:
        delta = attn_bwd_delta(o, dout)
    dq = torch.empty_like(q, memory_format=torch.contiguous_format) if need_dq else None
    dk = torch.empty_like(k, memory_format=torch.contiguous_format) if need_dkv else None
    dv = torch.empty_like(v, memory_format=torch.contiguous_format) if need_dkv else None
    nkb = -(-lk // block)
    lists = offs = None
    kk = 0
    if idx is not None:
        idx = _last_contig(idx)
        assert idx.dtype == torch.int32 and idx.shape[:3] == (b, h, -(-lq // block))
        kk = idx.shape[3]
        if need_dkv:
            lists, offs = key_lists if key_lists is not None else key_block_lists(idx, nkb)
            if key_lists is not None and (check_lists if check_lists is not None else os.environ.get("S3R_CHECK_LISTS") == "1"):
                if not key_lists_ascending(lists, offs):
                    raise ValueError("attn_bwd: key_lists must be ascending within every key block's group "
                                     "(build them with key_block_lists)")

    def st(t):
        return (t.stride(0), t.stride(1), t.stride(2)) if t is not None else (0, 0, 0)

    with torch.cuda.device(q.device):
        rc = _lib.lib().s3r_attn_bwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), dout.data_ptr(), lse.data_ptr(), delta.data_ptr(),
            idx.data_ptr() if idx is not None else None,
            lists.data_ptr() if lists is not None else None, offs.data_ptr() if offs is not None else None,
            lists.shape[-1] if lists is not None else 0,
            dq.data_ptr() if dq is not None else None, dk.data_ptr() if dk is not None else None,
            dv.data_ptr() if dv is not None else None,
            b, h, lq, lk, d, block, kk,
            *st(q), *st(k), *st(v), *st(dout), *st(dq), *st(dk), *st(dv), *st(idx),
            scale, _code(q), _stream(q))
    _lib.check(rc, "s3r_attn_bwd")
    return dq, dk, dv


class _SelectAttnFn(torch.autograd.Function):
    """Selection attention with gradients (reference TopkBlockSparseAttention, topk_blocksparse_attention.py:1041-1090)."""

    @staticmethod
    def forward(ctx, q, k, v, idx, block, softmax_scale):
        with torch.no_grad():
            o, lse = select_attn(q, k, v, idx, block, softmax_scale, return_lse=True)
        ctx.save_for_backward(q, k, v, o, lse, idx)
        ctx.block, ctx.scale = block, softmax_scale
        return o

    @staticmethod
    def backward(ctx, dout):
        q, k, v, o, lse, idx = ctx.saved_tensors
        dq, dk, dv = attn_bwd(q, k, v, o, dout, lse, idx, ctx.block, ctx.scale,
                              need_dq=ctx.needs_input_grad[0], need_dkv=ctx.needs_input_grad[1] or ctx.needs_input_grad[2])
        return dq, dk, dv, None, None, None


class _CompressedAttnFn(torch.autograd.Function):
    """Compressed attention + top-k with gradients for the attention output (the indices carry none; reference
    FlashAttnTopkFunc, flash_attention_topk.py:633-665)."""

    @staticmethod
    def forward(ctx, q, k, v, topk, softmax_scale, causal=False):
        with torch.no_grad():
            o, idx, lse = compressed_attn_topk(q, k, v, topk, softmax_scale, return_lse=True, causal=causal)
        ctx.save_for_backward(q, k, v, o, lse)
        ctx.scale = softmax_scale
        if idx is not None:
            ctx.mark_non_differentiable(idx)
        return o, idx

    @staticmethod
    def backward(ctx, dout, _didx):
        q, k, v, o, lse = ctx.saved_tensors
        dq, dk, dv = attn_bwd(q, k, v, o, dout, lse, None, 64, ctx.scale,
                              need_dq=ctx.needs_input_grad[0], need_dkv=ctx.needs_input_grad[1] or ctx.needs_input_grad[2])
        return dq, dk, dv, None, None, None   # (the reference's backward does not know of `causal` either, :653-666)


def _wants_grad(*ts: torch.Tensor) -> bool:
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in ts)


def select_attn_autograd(q, k, v, idx, block, softmax_scale=None):
    """:func:`select_attn`, differentiable in q, k, v where the backward kernels are built."""
    if not _wants_grad(q, k, v):
        return select_attn(q, k, v, idx, block, softmax_scale)
    if block in (128, 256):
        assert idx.shape[2] == -(-q.shape[2] // block), "topk_idx does not match the number of query blocks"
        idx, block = _as_64_token_blocks(idx, block, q.shape[2]), 64
    if not bwd_supported(q, block):
        raise RuntimeError("speed3r_amd: the attention backward is built for bf16/fp16, head_dim 64, blocks of 64 or 16 tokens")
    return _SelectAttnFn.apply(q, k, v, idx, block, softmax_scale)


def compressed_attn_topk_autograd(q, k, v, topk, softmax_scale=None, causal=False):
    """:func:`compressed_attn_topk` (``(o, idx)``), differentiable in q, k, v where the backward kernels are built."""
    if not _wants_grad(q, k, v):
        return compressed_attn_topk(q, k, v, topk, softmax_scale, causal=causal)
    if not bwd_supported(q):
        raise RuntimeError("speed3r_amd: the attention backward is built for bf16/fp16, head_dim 64 only")
    return _CompressedAttnFn.apply(q, k, v, topk, softmax_scale, causal)


_SIDE_STREAMS = {}


def _side_stream(device: torch.device) -> "torch.cuda.Stream":
    """One extra stream per device (default priority), created on first use and kept."""
    key = torch.device(device).index if torch.device(device).index is not None else torch.cuda.current_device()
    if key not in _SIDE_STREAMS:
        _SIDE_STREAMS[key] = torch.cuda.Stream(device=key)
    return _SIDE_STREAMS[key]


def _two_kernel_compressed(q: torch.Tensor, topk: int, block: int = 1) -> bool:
    """True where the compressed branch is two independent kernels (attention, indices without a score buffer).
    ``q``: the pooled queries (``block`` = 1) or the full tokens that will be pooled over ``block`` tokens."""
    return (q.dtype != torch.float32 and q.shape[-1] == 64 and topk in (1, 2, 4, 8, 16, 32)
            and -(-q.shape[2] // block) <= (1 << 21) and _lib.lib_has_fused_topk())


def topk_indices_on_side_stream(qc: torch.Tensor, kc: torch.Tensor, topk: int, softmax_scale: Optional[float] = None):
    """Launch the index kernel (top-k columns of the raw scores ``qc kc^T``, no score buffer) on the device's side
    stream, ordered after the work already queued on the current stream.  Returns ``(idx, join)``; call ``join()``
    on the current stream before the first use of ``idx`` there.  Needs :func:`_two_kernel_compressed`."""
    main = torch.cuda.current_stream(qc.device)
    side = _side_stream(qc.device)
    ready = torch.cuda.Event()
    ready.record(main)
    side.wait_event(ready)
    with torch.cuda.stream(side):
        _, idx = compressed_attn_topk(qc, kc, None, topk, softmax_scale)
        done = torch.cuda.Event()
        done.record(side)

    def join():
        torch.cuda.current_stream(qc.device).wait_event(done)
        idx.record_stream(torch.cuda.current_stream(qc.device))

    return idx, join


def sparse_global_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gate: torch.Tensor,
                            block: int = 64, topk: int = 16, softmax_scale: Optional[float] = None,
                            return_parts: bool = False, materialize_scores: Optional[bool] = None,
                            fuse_merge: bool = True, overlap: Optional[bool] = None, timeline: Optional[dict] = None):
    """The whole path on post-norm/RoPE q, k, v ``[B,H,N,D]`` and gate ``[B,H,N,2]``:
    pool -> compressed attention + top-k -> selection attention -> gated merge -> ``[B,N,H*D]``.
    The merge runs in the selection kernel's epilogue where the library offers it (same bits either way);
    ``return_parts`` needs the selection output and therefore runs the two operators separately.

    ``overlap`` (default: on where it applies): the indices need pooled q and k only, the compressed attention output
    is not read before the merge.  Where the two come from different kernels (no score buffer), the index kernel runs
    on a second stream next to the pooling of v and the compressed attention (same kernels, same results; only the
    schedule differs).  The index kernel alone leaves most of the chip idle below a few thousand pooled tokens (one
    workgroup per 128 pooled rows and head); measured at 266 496 tokens: 0.51 against 0.55 ms for everything in front
    of the selection kernel.  ``overlap=False`` runs the kernels one after the other on the calling stream.

    ``timeline``: a dict that receives timing events of the calling stream under "start", "pooled" (sequential
    schedule only), "select" (everything before the selection kernel is done) and "end".
    """
    def mark(name):
        if timeline is not None:
            ev = torch.cuda.Event(enable_timing=True)
            ev.record(torch.cuda.current_stream(q.device))
            timeline[name] = ev

    mark("start")
    if overlap is not False and materialize_scores is not True and not return_parts and q.is_cuda \
            and _two_kernel_compressed(q, topk, block):
        qc, kc = pool_mean(q, block), pool_mean(k, block)
        idx, join = topk_indices_on_side_stream(qc, kc, topk, softmax_scale)
        vc = pool_mean(v, block)
        o_cmp, _ = compressed_attn_topk(qc, kc, vc, None, softmax_scale)
        join()
    else:
        qc, kc, vc = pool_mean(q, block), pool_mean(k, block), pool_mean(v, block)
        mark("pooled")
        o_cmp, idx = compressed_attn_topk(qc, kc, vc, topk, softmax_scale, materialize_scores=materialize_scores)
    mark("select")
    if fuse_merge and not return_parts:
        out = select_attn_merge(q, k, v, idx, o_cmp, gate, block, softmax_scale)
        if out is not None:
            mark("end")
            return out
    o_sel = select_attn(q, k, v, idx, block, softmax_scale)
    mark("merge")
    out = gated_merge(o_cmp, o_sel, gate, block)
    mark("end")
    if return_parts:
        return out, dict(idx=idx, o_cmp=o_cmp, o_sel=o_sel, qc=qc, kc=kc, vc=vc)
    return out
