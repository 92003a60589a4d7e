"""CPU oracle for the global top-k block-sparse attention path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``speed3r_amd/`` imports this package;
only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` do, and there only as the checker / the timed CPU baseline.
"""
from .sparse_attention_oracle import (  # noqa: F401
    sortable_key,
    composite_keys,
    topk_from_scores,
    topk_streaming,
    pool_mean,
    compressed_scores,
    compressed_attention,
    flash_attn_topk,
    select_attention,
    select_attention_dense_masked,
    gated_merge,
    sparse_global_attention,
)
from .sparse_layer_oracle import rope2d, block_positions, sparse_layer  # noqa: F401,E402
from .model_oracle import pi3_sparse_like_forward  # noqa: F401,E402
from .attention_grad_oracle import (  # noqa: F401,E402
    select_attention_grads_autograd,
    compressed_attention_grads_autograd,
    attention_grads_formula,
    block_multiplicity,
    key_block_lists,
)
