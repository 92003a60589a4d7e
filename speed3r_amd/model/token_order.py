"""Tile-major token order of the reference model's decoder.

The reference reorders every frame's patch tokens so that each run of ``tile * tile`` consecutive tokens is one
``tile x tile`` square of the patch grid (pi3/models/pi3_sparse.py:29-45, applied to the tokens and to their positions
at :228-229 with ``sparse_block_size = 4``, undone at :265-269 by :47-71): a 16-token block of the sparse attention
(``block_size = 4`` -> 16 tokens, pi3/models/layers/sparse_attention.py:73,98) is then a 4 x 4 patch neighbourhood.

Token (y, x) of a ``gh x gw`` grid, row-major index ``y * gw + x``, moves to index
``((y // tile) * (gw // tile) + x // tile) * tile * tile + (y % tile) * tile + x % tile``.
"""
from __future__ import annotations

from torch import Tensor


def tile_major(x: Tensor, gh: int, gw: int, tile: int) -> Tensor:
    """``[B, gh*gw, C]`` row-major -> tile-major (one copy)."""
    assert gh % tile == 0 and gw % tile == 0, f"a {gh} x {gw} patch grid does not split into {tile} x {tile} tiles"
    b, n, c = x.shape
    assert n == gh * gw
    return x.reshape(b, gh // tile, tile, gw // tile, tile, c).permute(0, 1, 3, 2, 4, 5).reshape(b, n, c)


def tile_major_inverse(x: Tensor, gh: int, gw: int, tile: int) -> Tensor:
    """tile-major ``[B, gh*gw, C]`` -> row-major (one copy)."""
    assert gh % tile == 0 and gw % tile == 0, f"a {gh} x {gw} patch grid does not split into {tile} x {tile} tiles"
    b, n, c = x.shape
    assert n == gh * gw
    return x.reshape(b, gh // tile, gw // tile, tile, tile, c).permute(0, 1, 3, 2, 4, 5).reshape(b, n, c)
