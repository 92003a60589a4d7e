"""MI355X (gfx950) implementation of Speed3R's global top-k block-sparse attention path."""
from .sparse_attn import (  # noqa: F401
    flash_attn_topk_func, topk_blocksparse_attention,
    pool_mean, pool_qkv_packed, compressed_attn_topk, topk_rows, select_attn, select_attn_merge, gated_merge, sparse_global_attention,
)

__all__ = [
    "flash_attn_topk_func", "topk_blocksparse_attention", "pool_mean", "pool_qkv_packed", "compressed_attn_topk",
    "topk_rows", "select_attn", "select_attn_merge", "gated_merge", "sparse_global_attention",
]
