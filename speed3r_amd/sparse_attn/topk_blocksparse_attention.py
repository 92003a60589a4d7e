"""Drop-in for the reference module ``pi3/models/sparse_attn/topk_blocksparse_attention.py``.

Only the public forward operator is provided: ``topk_blocksparse_attention`` (reference
topk_blocksparse_attention.py:1093-1121).  Tensors are ``[batch, nheads, seq_len, head_dim]``
and ``topk_idx`` is int32 ``[batch, nheads, seq_len // block_size, topk]`` in block units, as
the reference kernel indexes them (:852-869).
"""
from __future__ import annotations

from typing import Optional

import torch

from . import ops


def topk_blocksparse_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, topk_idx: torch.Tensor,
                               block_size: int, softmax_scale: Optional[float] = None) -> torch.Tensor:
    """Every ``block_size``-row query block attends to the key blocks its ``topk_idx`` row lists.

    ``-1`` (or any index whose block starts at or beyond ``seq_len``) means "skip".  Returns the
    attention output with q's shape and dtype.  Blocks of 128 and 256 tokens run on the 64-token kernels: the same
    list serves the 2 (4) 64-row parts of a query block and a listed key block is visited as its 2 (4) 64-token parts.  The reference accepts bf16/fp16 only; fp32 is
    accepted here as well.  ``softmax_scale`` defaults to ``1/sqrt(head_dim)``.
    """
    assert q.dtype in (torch.bfloat16, torch.float16, torch.float32)
    assert q.dtype == k.dtype and k.dtype == v.dtype
    assert topk_idx.dtype == torch.int32
    assert block_size in {4, 16, 32, 64, 128, 256}
    batch, nheads, seq_len, _ = q.shape
    assert topk_idx.shape[0] == batch
    assert topk_idx.shape[1] == nheads
    assert topk_idx.shape[2] == -(-seq_len // block_size)
    return ops.select_attn_autograd(q, k, v, topk_idx, block_size, softmax_scale)
