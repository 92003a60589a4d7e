from .flash_attention_topk import flash_attn_topk_func  # noqa: F401
from .topk_blocksparse_attention import topk_blocksparse_attention  # noqa: F401
from .ops import (  # noqa: F401
    pool_mean, pool_qkv_packed, compressed_attn_topk, topk_rows, select_attn, select_attn_merge, gated_merge, sparse_global_attention,
)
