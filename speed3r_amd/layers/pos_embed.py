"""2-D rotary position embedding with the reference's numerics (pi3/models/layers/pos_embed.py:112-159).

The head dimension is split into a y half and an x half; each half gets a 1-D rotary embedding by the
token's y (resp. x) coordinate with frequencies ``base ** (-2 i / (D/2))`` and the "rotate half" pairing
(element j of a half is paired with element j + D/4).  The reference rounds the angles to the token dtype
before taking cos/sin and evaluates the products and the sum in the token dtype; this module keeps those
rounding points so that bf16 results agree with it, but builds the angles straight from the positions
(no per-length tables).
"""
from __future__ import annotations

import torch
from torch import nn


class RoPE2D(nn.Module):
    def __init__(self, freq: float = 100.0, F0: float = 1.0, max_positions: int = 0) -> None:
        super().__init__()
        self.base = freq
        self.F0 = F0
        # number of rows of the cos/sin tables the fused kernel reads; 0: sized from the positions of every call
        # (one device synchronisation per call, like the reference's ``positions.max()``)
        self.max_positions = max_positions
        self._tables = {}

    def tables(self, head_dim: int, n_pos: int, device, dtype):
        """cos, sin ``[n_pos, head_dim // 4]`` in ``dtype``: row p holds cos/sin of the angles ``p * inv_freq`` after
        their rounding to ``dtype`` (the reference's table, pos_embed.py:121-131, without the duplicated half)."""
        key = (head_dim, n_pos, str(device), dtype)
        if key not in self._tables:
            half = head_dim // 2
            inv_freq = 1.0 / (self.base ** (torch.arange(0, half, 2, device=device, dtype=torch.float32) / half))
            t = torch.arange(n_pos, device=device, dtype=torch.float32)
            ang = torch.einsum("i,j->ij", t, inv_freq).to(dtype)
            self._tables[key] = (ang.cos().contiguous(), ang.sin().contiguous())
        return self._tables[key]

    def _cos_sin(self, pos1d: torch.Tensor, half: int, dtype: torch.dtype):
        # pos1d [B, N] integer coordinates -> cos, sin [B, 1, N, half] with the two quarters holding the same angles
        quarter = half // 2
        inv_freq = 1.0 / (self.base ** (torch.arange(0, half, 2, device=pos1d.device, dtype=torch.float32) / half))
        ang = (pos1d.to(torch.float32)[..., None] * inv_freq).to(dtype)            # rounded like the reference's table
        assert ang.shape[-1] == quarter
        ang = torch.cat((ang, ang), dim=-1)[:, None]
        return ang.cos(), ang.sin()

    @staticmethod
    def _rotate(t: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
        a, b = t.chunk(2, dim=-1)
        return t * cos + torch.cat((-b, a), dim=-1) * sin

    def forward(self, tokens: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """tokens [B, H, N, D], positions [B, N, 2] (y, x) integers -> rotated tokens, same shape and dtype."""
        assert tokens.shape[-1] % 4 == 0, "head_dim must be a multiple of four"
        assert positions.ndim == 3 and positions.shape[-1] == 2, "positions must be [B, N, 2]"
        half = tokens.shape[-1] // 2
        y, x = tokens.chunk(2, dim=-1)
        cy, sy = self._cos_sin(positions[..., 0], half, tokens.dtype)
        cx, sx = self._cos_sin(positions[..., 1], half, tokens.dtype)
        return torch.cat((self._rotate(y, cy, sy), self._rotate(x, cx, sx)), dim=-1)


def block_positions(xpos: torch.Tensor, block: int) -> torch.Tensor:
    """Position of every ``block``-token block: the truncated mean of its tokens' positions
    (pi3/models/layers/sparse_attention.py:107-108); a ragged last block averages its valid tokens."""
    b, n, two = xpos.shape
    nc = -(-n // block)
    pad = nc * block - n
    xf = xpos.to(torch.float32)
    if pad:
        xf = torch.cat((xf, xf.new_zeros((b, pad, two))), dim=1)
    sums = xf.view(b, nc, block, two).sum(dim=2)
    counts = torch.full((nc,), float(block), device=xpos.device)
    if pad:
        counts[-1] = float(block - pad)
    return (sums / counts[None, :, None]).to(torch.int32)
