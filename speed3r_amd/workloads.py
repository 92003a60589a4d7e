"""Seeded synthetic inputs of the benchmark configurations (operator level).

All tensors are generated on the CPU with a fixed ``torch.Generator`` seed, so the HIP path
and any CPU checker see identical bits.  Layout ``[B, H, N, D]`` contiguous; ``B=1, H=16,
D=64, block=64`` throughout; 1041 tokens per frame.

  config 1: 8 frames   (N=8 328, ragged tail 8), fp32, N(0,1)/8, seed 0
  config 2: 64 frames  (N=66 624),  bf16, N(0,1)/8, seed 1
  config 3: 256 frames (N=266 496), bf16, N(0,1)/8 + per-frame low-rank component, seed 3
  config 4: 1000 frames (N=1 041 000, ragged tail 40), bf16, same generator as config 3

Low-rank component (configs 3, 4): per head a basis ``W[h] in R^{8x64} ~ N(0,1)/sqrt(8)``; per
(head, frame) coefficients ``c ~ N(0, 0.5^2)``; ``u[h,f] = c[h,f] W[h]`` is added to every q and
k token of frame f (same u for both, so same-frame and aligned-frame blocks score higher) and
an independent draw ``u_v`` to v.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict

import torch

TOKENS_PER_FRAME = 1041
HEADS = 16
HEAD_DIM = 64
BLOCK = 64


@dataclass(frozen=True)
class Config:
    name: str
    frames: int
    dtype: torch.dtype
    seed: int
    low_rank: bool
    topk: int = 16

    @property
    def tokens(self) -> int:
        return self.frames * TOKENS_PER_FRAME


CONFIGS: Dict[str, Config] = {
    "cfg1": Config("cfg1_8f_fp32", 8, torch.float32, 0, False),
    "cfg2": Config("cfg2_64f_bf16", 64, torch.bfloat16, 1, False),
    "cfg3": Config("cfg3_256f_bf16", 256, torch.bfloat16, 3, True),
    "cfg4": Config("cfg4_1000f_bf16", 1000, torch.bfloat16, 3, True),
}


def make_qkv(frames: int, dtype: torch.dtype, seed: int, low_rank: bool, heads: int = HEADS,
             head_dim: int = HEAD_DIM, tokens_per_frame: int = TOKENS_PER_FRAME, head_chunk: int = 4):
    """Returns q, k, v ``[1, heads, frames*tokens_per_frame, head_dim]`` (CPU, ``dtype``)."""
    g = torch.Generator().manual_seed(seed)
    n = frames * tokens_per_frame
    out = [torch.empty((1, heads, n, head_dim), dtype=dtype) for _ in range(3)]
    if low_rank:
        rank = 8
        w = torch.randn((heads, rank, head_dim), generator=g) / rank ** 0.5
        c_qk = torch.randn((heads, frames, rank), generator=g) * 0.5
        c_v = torch.randn((heads, frames, rank), generator=g) * 0.5
        u_qk = torch.bmm(c_qk, w)  # [heads, frames, head_dim]
        u_v = torch.bmm(c_v, w)
    for h0 in range(0, heads, head_chunk):
        h1 = min(heads, h0 + head_chunk)
        for which in range(3):
            x = torch.randn((h1 - h0, n, head_dim), generator=g) / 8.0
            if low_rank:
                u = (u_v if which == 2 else u_qk)[h0:h1]
                x = (x.view(h1 - h0, frames, tokens_per_frame, head_dim) + u[:, :, None, :]).view(h1 - h0, n, head_dim)
            out[which][0, h0:h1] = x.to(dtype)
    return tuple(out)


def make_qkv_on_device(frames: int, dtype: torch.dtype, seed: int, low_rank: bool, device, heads: int = HEADS,
                       head_dim: int = HEAD_DIM, tokens_per_frame: int = TOKENS_PER_FRAME):
    """The generator of :func:`make_qkv` drawn on ``device`` from that device's own seeded stream: the same
    distribution (noise plus per-frame low-rank component), other bits.  For timing runs that need no CPU checker."""
    g = torch.Generator(device=device).manual_seed(seed)
    n = frames * tokens_per_frame
    out = []
    if low_rank:
        rank = 8
        w = torch.randn((heads, rank, head_dim), generator=g, device=device) / rank ** 0.5
        u_qk = torch.bmm(torch.randn((heads, frames, rank), generator=g, device=device) * 0.5, w)
        u_v = torch.bmm(torch.randn((heads, frames, rank), generator=g, device=device) * 0.5, w)
    for which in range(3):
        t = torch.empty((1, heads, n, head_dim), dtype=dtype, device=device)
        for h in range(heads):   # one head at a time: the fp32 draw of a whole tensor would double the footprint
            x = torch.randn((n, head_dim), generator=g, device=device) / 8.0
            if low_rank:
                u = (u_v if which == 2 else u_qk)[h]
                x = (x.view(frames, tokens_per_frame, head_dim) + u[:, None, :]).view(n, head_dim)
            t[0, h] = x.to(dtype)
        out.append(t)
    return tuple(out)


def make_gate(n: int, dtype: torch.dtype, seed: int, heads: int = HEADS) -> torch.Tensor:
    """Gate ``[1, heads, n, 2] = sigmoid(N(0,1))`` from its own seeded stream."""
    g = torch.Generator().manual_seed(seed + 1000)
    return torch.sigmoid(torch.randn((1, heads, n, 2), generator=g)).to(dtype)


def make_config(name: str):
    """Returns (cfg, q, k, v, gate) for ``name`` in CONFIGS."""
    cfg = CONFIGS[name]
    q, k, v = make_qkv(cfg.frames, cfg.dtype, cfg.seed, cfg.low_rank)
    gate = make_gate(cfg.tokens, cfg.dtype, cfg.seed)
    return cfg, q, k, v, gate


def selection_flops(n: int, topk: int, heads: int = HEADS, head_dim: int = HEAD_DIM, block: int = BLOCK) -> float:
    """QK^T + PV multiply-adds of the selection branch, 2 FLOP each: 4 N K block D H."""
    return 4.0 * n * topk * block * head_dim * heads


def compressed_flops(n: int, heads: int = HEADS, head_dim: int = HEAD_DIM, block: int = BLOCK) -> float:
    nc = -(-n // block)
    return 4.0 * nc * nc * head_dim * heads
