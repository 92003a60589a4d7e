"""Pins of the oracle's causal variants (flash_attention_topk.py:71,93; the reference layer never takes them).

Attention: ``F.scaled_dot_product_attention(is_causal=True)`` (a library routine with the same top-left aligned
mask).  Indices: a per-row Python sort over (score descending, column ascending) with the keys above the diagonal at
-inf, hand-made known answers, and mistakes a restatement could plausibly make (masked keys left out instead of
ranked last, a mask aligned bottom-right) that must change the result."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from oracle import sparse_attention_oracle as so


def _qkv(lq, lk, seed, h=2, d=64):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn((1, h, lq, d), generator=g), torch.randn((1, h, lk, d), generator=g),
            torch.randn((1, h, lk, d), generator=g))


@pytest.mark.parametrize("lq,lk", [(150, 150), (64, 64), (100, 180), (130, 70), (1, 5)])
def test_causal_attention_is_the_library_routine(lq, lk):
    q, k, v = _qkv(lq, lk, 3)
    o, lse, s = oracle.compressed_attention(q, k, v, causal=True, out_dtype=torch.float32)
    want = F.scaled_dot_product_attention(q, k, v, is_causal=True)
    assert (o - want).abs().max().item() <= 2e-6
    z = (q @ k.transpose(-1, -2)) / math.sqrt(64)
    keep = torch.arange(lk)[None, :] <= torch.arange(lq)[:, None]
    want_lse = torch.logsumexp(z.masked_fill(~keep, float("-inf")), dim=-1)
    assert (lse - want_lse).abs().max().item() <= 2e-6
    assert torch.equal(torch.isinf(s) & (s < 0), ~keep.expand_as(s))        # the scores carry the mask ...
    assert torch.equal(s[keep.expand_as(s)], (q @ k.transpose(-1, -2))[keep.expand_as(s)])   # ... and nothing else


def _by_sort(raw, k, mistake=None):
    """Row i: columns ordered by (score descending, column ascending), keys above the diagonal at -inf."""
    lq, lk = raw.shape
    out = np.empty((lq, k), dtype=np.int32)
    for i in range(lq):
        if mistake == "bottom_right":
            seen = lambda j: j <= i + (lk - lq)
        else:
            seen = lambda j: j <= i
        cand = [j for j in range(lk) if seen(j)] if mistake == "left_out" else list(range(lk))
        order = sorted(cand, key=lambda j: (-(raw[i, j] if seen(j) else -math.inf), j))[:k]
        order += [lk - 1] * (k - len(order))
        out[i] = order
    return out


@pytest.mark.parametrize("lq,lk,k", [(150, 150, 16), (200, 200, 64), (100, 180, 8), (130, 70, 32), (40, 40, 64), (3, 2, 4)])
def test_causal_indices_are_a_sort_over_the_masked_row(lq, lk, k):
    q, kk, v = _qkv(lq, lk, 11, h=1)
    _, _, s = oracle.compressed_attention(q, kk, v, causal=True)
    got = so.topk_from_scores_causal(s, k)[0, 0]
    raw = (q @ kk.transpose(-1, -2))[0, 0].numpy()
    np.testing.assert_array_equal(got, _by_sort(raw, k))   # (fewer keys than slots: the filler is the last column)
    _, idx = oracle.flash_attn_topk(q, kk, v, k, causal=True)
    np.testing.assert_array_equal(idx[0, 0].numpy(), got)


def test_causal_indices_known_answers():
    lq = lk = 200
    q, kk, v = _qkv(lq, lk, 5, h=1)
    _, _, s = oracle.compressed_attention(q, kk, v, causal=True)
    idx = so.topk_from_scores_causal(s, 4)[0, 0]
    np.testing.assert_array_equal(idx[0], [0, 1, 2, 3])           # one visible key, then the masked ones, lowest column first
    raw = (q @ kk.transpose(-1, -2))[0, 0]
    first_two = sorted([0, 1], key=lambda j: -raw[1, j].item())
    np.testing.assert_array_equal(idx[1], first_two + [2, 3])
    assert (idx[150] <= 150).all() and len(set(idx[150].tolist())) == 4
    np.testing.assert_array_equal(np.sort(idx[150]), np.sort(torch.topk(raw[150, :151], 4).indices.numpy()))


def test_plausible_mistakes_change_the_indices():
    q, kk, v = _qkv(100, 180, 7, h=1)
    raw = (q @ kk.transpose(-1, -2))[0, 0].numpy()
    right = _by_sort(raw, 8)
    assert (right != _by_sort(raw, 8, "left_out")).any()          # masked keys are ranked (last), not dropped
    assert (right != _by_sort(raw, 8, "bottom_right")).any()      # the mask is aligned with row 0 / column 0
    _, _, s = oracle.compressed_attention(q, kk, v, causal=True)
    np.testing.assert_array_equal(so.topk_from_scores_causal(s, 8)[0, 0], right)
    assert (oracle.topk_from_scores(torch.from_numpy(raw)[None, None], 8)[0, 0] != right).any()   # and causal is not a no-op
