"""Drop-in for the reference module ``pi3/models/sparse_attn/flash_attention_topk.py``.

Only the public forward operator is provided: ``flash_attn_topk_func`` (reference
``FlashAttnTopkFunc.apply``, flash_attention_topk.py:633-668).  Arguments keep the reference's
names, order and meaning; tensors are ``[batch, nheads, seqlen, headdim]`` (the layout the
reference kernel actually indexes, flash_attention_topk.py:159).
"""
from __future__ import annotations

from . import ops

_BLOCK_N = 64        # reference tile constants (flash_attention_topk.py:165-167)
_BLOCK_HEADDIM = 64


def flash_attn_topk_func(q, k, v, topk_val, bias=None, causal=False, softmax_scale=None):
    """Compressed-branch attention and top-k block selection.

    Returns ``(o, topk_indices)``: ``o`` has q's shape and dtype; ``topk_indices`` is int32
    ``[batch, nheads, seqlen_q, topk_val]`` holding, for every query row, the columns of the
    ``topk_val`` largest raw (unscaled) fp32 scores in descending order, equal scores lowest
    column first.  ``bias`` is unused by the reference kernel and must be None; the causal
    variant is never taken by the reference layer and is not provided.
    """
    headdim = q.shape[-1]
    assert topk_val <= _BLOCK_N, f"Top-K value ({topk_val}) cannot exceed BLOCK_N ({_BLOCK_N})"
    assert headdim <= _BLOCK_HEADDIM, "headdim must be less than or equal to BLOCK_HEADDIM"
    assert topk_val >= 1 and (topk_val & (topk_val - 1)) == 0, "Top-K value must be a power of two"
    if bias is not None:
        raise NotImplementedError("flash_attn_topk_func: bias is not supported (the reference kernel ignores it)")
    if causal:
        raise NotImplementedError("flash_attn_topk_func: the causal variant is not provided")
    o, idx = ops.compressed_attn_topk_autograd(q, k, v, topk_val, softmax_scale)
    return o, idx
