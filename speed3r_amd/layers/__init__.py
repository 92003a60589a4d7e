from .pos_embed import RoPE2D, block_positions  # noqa: F401
from .sparse_attention import SparseFlashAttentionRope  # noqa: F401
