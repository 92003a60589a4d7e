"""The tile-major token order of the reference model's decoder (pi3/models/pi3_sparse.py:29-71) against the index
formula written out with plain loops: bit-exact, both directions, for tokens and for their positions."""
import pytest
import torch

import oracle
from oracle.model_oracle import tile_major_index
from speed3r_amd.model.token_order import tile_major, tile_major_inverse


def _place(y, x, gw, tile):
    return ((y // tile) * (gw // tile) + x // tile) * tile * tile + (y % tile) * tile + x % tile


@pytest.mark.parametrize("gh,gw,tile", [(4, 4, 4), (8, 12, 4), (36, 28, 4), (6, 4, 2), (3, 5, 1)])
def test_tile_major_order_matches_the_index_formula(gh, gw, tile):
    g = torch.Generator().manual_seed(gh * 100 + gw)
    x = torch.randn((3, gh * gw, 5), generator=g)
    got = tile_major(x, gh, gw, tile)
    want = torch.empty_like(x)
    for y in range(gh):
        for xx in range(gw):
            want[:, _place(y, xx, gw, tile)] = x[:, y * gw + xx]
    assert torch.equal(got, want)
    assert torch.equal(tile_major_inverse(got, gh, gw, tile), x)
    # the oracle's gather index says the same
    assert torch.equal(x[:, tile_major_index(gh, gw, tile)], want)
    # every run of tile*tile tokens is one tile of the grid: positions inside a run span a tile x tile square
    yy, xg = torch.meshgrid(torch.arange(gh), torch.arange(gw), indexing="ij")
    pos = torch.stack((yy, xg), dim=-1).reshape(1, gh * gw, 2)
    runs = tile_major(pos, gh, gw, tile).view(gh * gw // (tile * tile), tile * tile, 2)
    assert ((runs.max(dim=1).values - runs.min(dim=1).values) == tile - 1).all()
    assert (runs.min(dim=1).values % tile == 0).all()


def test_tile_major_rejects_grids_that_do_not_split():
    with pytest.raises(AssertionError):
        tile_major(torch.zeros(1, 37 * 28, 2), 37, 28, 4)      # 518 x 392 frames: 37 patch rows
