"""CPU restatement of the reference's global sparse attention LAYER around the operators.

TEST INFRASTRUCTURE ONLY -- never imported by the product package.

Follows, in eager PyTorch on the CPU (paths relative to the reference root):

  rope2d             pi3/models/layers/pos_embed.py:112-159  (table of angles per integer position, rounded to the
                     token dtype, cos/sin of the rounded angles, "rotate half" pairing, y half then x half)
  block_positions    pi3/models/layers/sparse_attention.py:107-108  (truncated mean position of a block)
  sparse_layer       pi3/models/layers/sparse_attention.py:90-141   (projection, gate, pooling of the raw projection,
                     qk-norm and RoPE on both branches, the two operators, merge, output projection)

The two operators, pooling and merge inside ``sparse_layer`` are the functions of ``sparse_attention_oracle``.

Pins (tests/test_oracle_layer.py): rope2d against the textbook rotation (for head_dim 4 every half is one plane
rotated by ``pos`` radians), against its invariants (position 0 is the identity, norms are preserved, the y half
ignores x, inner products depend on position differences only) and, in fp64, against a complex-number
formulation written independently; block_positions against hand-computed cases.  ``sparse_layer``
(tests/test_oracle_layer_composition.py): with every key block selected the layer must equal
``proj(g0 * broadcast(compressed row) + g1 * dense attention)`` built from explicit per-head row ranges of the weight
matrices, ``F.layer_norm``, ``F.scaled_dot_product_attention``, a complex-number rotation and plain block means; with
fewer blocks, the block-masked dense softmax under ``torch.topk`` of the pooled scores; gate extremes isolate each
branch (the (0, 1) extreme is the reference's eager dense layer, sparse_attention.py:39-58).  Each check also asserts
that ten plausible mistakes (swapped split order, swapped gate pairing, norm before pooling, rounded or first-token
block positions, exchanged y/x, ...) land far outside the tolerance.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F

from . import sparse_attention_oracle as ops


def rope2d(tokens: torch.Tensor, positions: torch.Tensor, base: float = 100.0) -> torch.Tensor:
    """tokens [B,H,N,D], positions [B,N,2] (y,x) -> tokens with the 2-D rotary embedding applied."""
    d_half = tokens.shape[-1] // 2
    seq = int(positions.max()) + 1
    inv_freq = 1.0 / (base ** (torch.arange(0, d_half, 2).float() / d_half))
    table = torch.einsum("i,j->ij", torch.arange(seq, dtype=torch.float32), inv_freq).to(tokens.dtype)
    table = torch.cat((table, table), dim=-1)
    cos_t, sin_t = table.cos(), table.sin()

    def rope1d(t, pos1d):
        cos = F.embedding(pos1d.long(), cos_t)[:, None]
        sin = F.embedding(pos1d.long(), sin_t)[:, None]
        t1, t2 = t[..., : t.shape[-1] // 2], t[..., t.shape[-1] // 2:]
        return t * cos + torch.cat((-t2, t1), dim=-1) * sin

    y, x = tokens.chunk(2, dim=-1)
    return torch.cat((rope1d(y, positions[..., 0]), rope1d(x, positions[..., 1])), dim=-1)


def block_positions(xpos: torch.Tensor, block: int) -> torch.Tensor:
    b, n, _ = xpos.shape
    nc = -(-n // block)
    out = torch.empty((b, nc, 2), dtype=torch.int32)
    for j in range(nc):
        out[:, j] = xpos[:, j * block:min(n, (j + 1) * block)].float().mean(dim=1).int()
    return out


def sparse_layer(x, w_qkv, b_qkv, w_gate, b_gate, w_proj, b_proj, num_heads: int, block: int, topk: int,
                 xpos: Optional[torch.Tensor] = None, qn_w=None, qn_b=None, kn_w=None, kn_b=None,
                 rope_base: float = 100.0, idx_override: Optional[torch.Tensor] = None, ln_eps: float = 1e-5):
    """One forward of the layer on CPU tensors of one dtype.  ``qn_*``/``kn_*``: LayerNorm(head_dim) affine
    parameters (None: no qk-norm), ``ln_eps`` their epsilon.  Returns dict(out, idx, o_cmp, o_sel)."""
    b, n, c = x.shape
    h, d = num_heads, c // num_heads
    dt = x.dtype
    qkv = F.linear(x, w_qkv, b_qkv)
    gate = torch.sigmoid(F.linear(x, w_gate, b_gate)).view(b, n, h, 2).permute(0, 2, 1, 3)

    def norm(t, w, bias):
        if w is None:
            return t
        return F.layer_norm(t.float(), (d,), w.float(), bias.float(), ln_eps).to(dt)

    q, k, v = qkv.view(b, n, 3, h, d).permute(2, 0, 3, 1, 4).unbind(0)
    qc, kc, vc = (ops.pool_mean(t, block, out_dtype=dt) for t in (q, k, v))
    qc, kc = norm(qc, qn_w, qn_b), norm(kc, kn_w, kn_b)
    if xpos is not None:
        pc = block_positions(xpos, block)
        qc, kc = rope2d(qc, pc, rope_base), rope2d(kc, pc, rope_base)
    o_cmp, idx = ops.flash_attn_topk(qc, kc, vc, topk)
    if idx_override is not None:
        idx = idx_override

    q, k = norm(q, qn_w, qn_b), norm(k, kn_w, kn_b)
    if xpos is not None:
        q, k = rope2d(q, xpos, rope_base), rope2d(k, xpos, rope_base)
    o_sel = ops.select_attention(q, k, v, idx, block, out_dtype=dt)
    merged = ops.gated_merge(o_cmp.to(dt), o_sel, gate, block)
    out = F.linear(merged, w_proj, b_proj)
    return dict(out=out, idx=idx, o_cmp=o_cmp, o_sel=o_sel)
