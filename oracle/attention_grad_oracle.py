"""CPU oracle of the attention backward (TEST INFRASTRUCTURE ONLY; see the package docstring).

The reference computes the gradients with hand-written kernels (backward_sum_o_do, backward_dkdv, backward_dq,
pi3/models/sparse_attn/topk_blocksparse_attention.py:132-170,558-712,722-850 and flash_attention_topk.py:204-630)
of the formulas
    P = exp(scale * Q K^T - lse),  dV = P^T dO,  dP = dO V^T,  dS = scale * P * (dP - rowsum(dO * O)),
    dQ = dS K,  dK = dS^T Q
over the (query block, key block) pairs of the index tensor.  Two restatements live here: ``attention_grads_formula``
evaluates exactly those formulas (dense, with per-pair multiplicities for the selection), and ``*_autograd`` lets
torch differentiate the forward oracle.  tests/test_oracle_grads.py pins them against each other, against autograd of
``F.scaled_dot_product_attention`` and against central differences in fp64.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

from .sparse_attention_oracle import compressed_attention, select_attention, select_attention_dense_masked


def select_attention_grads_autograd(q, k, v, idx, block: int, dout, softmax_scale: Optional[float] = None,
                                    brute_force: bool = False) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dq, dk, dv) of the selection attention by torch autograd through the forward oracle (fp32 gather path, or
    the fp64 dense brute force for tiny shapes)."""
    dt = torch.float64 if brute_force else torch.float32
    qq, kk, vv = (t.detach().to(dt).requires_grad_(True) for t in (q, k, v))
    if brute_force:
        o = select_attention_dense_masked(qq, kk, vv, idx, block, softmax_scale)
    else:
        o = select_attention(qq, kk, vv, idx, block, softmax_scale, out_dtype=torch.float32)
    o.backward(dout.to(o.dtype))
    return qq.grad, kk.grad, vv.grad


def compressed_attention_grads_autograd(q, k, v, dout, softmax_scale: Optional[float] = None):
    """(dq, dk, dv) of the dense attention over pooled tokens by autograd through the forward oracle (fp32)."""
    qq, kk, vv = (t.detach().to(torch.float32).requires_grad_(True) for t in (q, k, v))
    o, _, _ = compressed_attention(qq, kk, vv, softmax_scale, out_dtype=torch.float32)
    o.backward(dout.to(torch.float32))
    return qq.grad, kk.grad, vv.grad


def attention_grads_formula(q, k, v, dout, mult: Optional[torch.Tensor] = None, softmax_scale: Optional[float] = None,
                            dtype: torch.dtype = torch.float64):
    """The reference's formulas, dense: q [.., Lq, D], k, v [.., Lk, D], dout like q; ``mult`` [.., Lq, Lk] gives how
    many times query i attends key j (0 = not at all; None = once each).  Returns (dq, dk, dv, o, lse)."""
    d = q.shape[-1]
    scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(d)
    qd, kd, vd, gd = (t.to(dtype) for t in (q, k, v, dout))
    s = (qd @ kd.transpose(-1, -2)) * scale
    if mult is None:
        mult = torch.ones_like(s)
    mult = mult.to(dtype)
    sm = torch.where(mult > 0, s, torch.full_like(s, -float("inf")))
    mx = sm.max(dim=-1, keepdim=True).values
    mx = torch.where(torch.isinf(mx), torch.zeros_like(mx), mx)
    den = (torch.exp(sm - mx) * mult).sum(dim=-1, keepdim=True)
    lse = mx + torch.log(den)                      # -inf for a row that attends nothing
    p = torch.where(mult > 0, torch.exp(sm - lse), torch.zeros_like(s)) * mult   # P with multiplicities
    p = torch.where(den > 0, p, torch.zeros_like(p))
    o = p @ vd
    delta = (gd * o).sum(dim=-1, keepdim=True)
    dv = p.transpose(-1, -2) @ gd
    dp = gd @ vd.transpose(-1, -2)
    ds = scale * p * (dp - delta)
    dq = ds @ kd
    dk = ds.transpose(-1, -2) @ qd
    return dq, dk, dv, o, lse.squeeze(-1)


def block_multiplicity(idx: torch.Tensor, n: int, block: int) -> torch.Tensor:
    """[B,H,N,N] multiplicities from block indices [B,H,ceil(N/block),K]: entries < 0 or starting at or beyond n are
    skipped, duplicates count twice (topk_blocksparse_attention.py:96-98)."""
    b, h, nqb, kk = idx.shape
    mult = torch.zeros((b, h, n, n), dtype=torch.float64)
    for bi in range(b):
        for hi in range(h):
            for m in range(nqb):
                r0, r1 = m * block, min(n, (m + 1) * block)
                for j in idx[bi, hi, m].tolist():
                    if j < 0 or j * block >= n:
                        continue
                    mult[bi, hi, r0:r1, j * block:min(n, (j + 1) * block)] += 1.0
    return mult


def key_block_lists(idx: torch.Tensor, n_key_blocks: int):
    """Plain-loop restatement of the key-centric lists (reference count_query_fixedlen / reorder_topk_idx_fixedlen,
    topk_blocksparse_attention.py:423-554): per (b, h) a list of lists, lists[j] = ascending query-block ids that
    name key block j, one entry per occurrence."""
    b, h, nqb, kk = idx.shape
    out = []
    for bi in range(b):
        for hi in range(h):
            lists = [[] for _ in range(n_key_blocks)]
            for m in range(nqb):
                for j in idx[bi, hi, m].tolist():
                    if 0 <= j < n_key_blocks:
                        lists[j].append(m)
            out.append(lists)
    return out
