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
    column first.

    ``bias`` is accepted and ignored, as in the reference (``FlashAttnTopkFunc.forward`` never hands it to
    ``forward_with_topk``, flash_attention_topk.py:646-648).  ``causal=True`` is the kernel's IS_CAUSAL variant
    (:71,93; the reference layer never asks for it): query i attends the keys j <= i and ranks the keys of the
    tiles its 64-row block visits, ``j < min((i // 64 + 1) * 64, seqlen_k)``, those above i with the score -inf.
    Its gradients are, as in the reference (:653-666), those of the non-causal operator on the causal
    log-sum-exp.
    """
    headdim = q.shape[-1]
    assert topk_val <= _BLOCK_N, f"Top-K value ({topk_val}) cannot exceed BLOCK_N ({_BLOCK_N})"
    assert headdim <= _BLOCK_HEADDIM, "headdim must be less than or equal to BLOCK_HEADDIM"
    assert topk_val >= 1 and (topk_val & (topk_val - 1)) == 0, "Top-K value must be a power of two"
    o, idx = ops.compressed_attn_topk_autograd(q, k, v, topk_val, softmax_scale, causal=bool(causal))
    return o, idx
