"""Shared test utilities (no reference code, no oracle logic)."""
import numpy as np
import torch


def from_bf16_bits(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def max_abs(a: torch.Tensor, b: torch.Tensor) -> float:
    return (a.double().cpu() - b.double().cpu()).abs().max().item()


def merged_within_rounding(got: torch.Tensor, o_cmp: torch.Tensor, o_sel: torch.Tensor, gate: torch.Tensor, block: int) -> bool:
    """``got`` [B,N,H*D] against gate0 * o_cmp[block of the row] + gate1 * o_sel evaluated in fp32, within the rounding
    steps that separate the ways of evaluating it in a 16-bit type: the eager expression rounds o_sel, both products and
    the sum, a fused evaluation rounds once.  Bound: four steps of the output type on |gate0 o_cmp| + |gate1 o_sel|
    (the terms, not the sum: they may cancel)."""
    b, h, n, d = o_sel.shape
    blk = torch.arange(n, device=o_sel.device) // block
    x = gate[..., 0:1].float() * o_cmp.float()[:, :, blk]
    y = gate[..., 1:2].float() * o_sel.float()
    want = (x + y).permute(0, 2, 1, 3).reshape(b, n, h * d)
    room = (x.abs() + y.abs()).permute(0, 2, 1, 3).reshape(b, n, h * d)
    step = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[got.dtype]
    return bool(((got.float() - want).abs() <= 4 * step * room + 1e-6).all())
