"""Pins of the oracle's floating-point stages (CPU): library routines, closed forms, brute force.

Reference lines restated by the oracle: pooling sparse_attention.py:97-99; compressed attention
flash_attention_topk.py:87-110,135-142; selection topk_blocksparse_attention.py:86-128; merge
sparse_attention.py:127-136.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from helpers import from_bf16_bits, max_abs


# ---------------------------------------------------------------- pooling
def test_pool_equals_avg_pool1d():
    g = torch.Generator().manual_seed(0)
    x = torch.randn((2, 3, 256, 16), generator=g)
    want = F.avg_pool1d(x.permute(0, 1, 3, 2).reshape(6, 16, 256), kernel_size=64, stride=64)
    want = want.reshape(2, 3, 16, 4).permute(0, 1, 3, 2)
    assert max_abs(oracle.pool_mean(x, 64), want) < 1e-6


def test_pool_ragged_tail_equals_ceil_mode_avg_pool():
    g = torch.Generator().manual_seed(1)
    x = torch.randn((1, 2, 200, 8), generator=g)
    want = F.avg_pool1d(x.permute(0, 1, 3, 2).reshape(2, 8, 200), kernel_size=64, stride=64, ceil_mode=True)
    want = want.reshape(1, 2, 8, 4).permute(0, 1, 3, 2)
    assert max_abs(oracle.pool_mean(x, 64), want) < 1e-6


def test_pool_closed_forms():
    const = torch.full((1, 1, 130, 4), 3.25)
    assert torch.equal(oracle.pool_mean(const, 64), torch.full((1, 1, 3, 4), 3.25))
    ramp = torch.arange(128, dtype=torch.float32).view(1, 1, 128, 1).expand(1, 1, 128, 4)
    got = oracle.pool_mean(ramp, 64)
    assert torch.allclose(got[0, 0, :, 0], torch.tensor([31.5, 95.5]))


def test_pool_fixture(golden):
    for name in ("q", "k", "v"):
        x = from_bf16_bits(golden[name])
        got = oracle.pool_mean(x, 64, out_dtype=torch.float32)
        assert max_abs(got, torch.from_numpy(golden[f"pooled_{name}"])) < 1e-6


# ---------------------------------------------------------------- compressed attention
def test_compressed_equals_sdpa_and_fp64():
    g = torch.Generator().manual_seed(2)
    q, k, v = (torch.randn((1, 2, 150, 64), generator=g) for _ in range(3))
    o, lse, s = oracle.compressed_attention(q, k, v)
    assert max_abs(o, F.scaled_dot_product_attention(q, k, v)) < 2e-6
    s64 = q.double() @ k.double().transpose(-1, -2)
    assert max_abs(s, s64) < 1e-4                       # raw, unscaled
    assert max_abs(lse, torch.logsumexp(s64 / 8.0, dim=-1)) < 1e-5
    assert max_abs(o, torch.softmax(s64 / 8.0, dim=-1) @ v.double()) < 2e-6


def test_compressed_invariants():
    g = torch.Generator().manual_seed(3)
    q = torch.randn((1, 1, 10, 64), generator=g)
    v = torch.randn((1, 1, 33, 64), generator=g)
    k_same = torch.randn((1, 1, 1, 64), generator=g).expand(1, 1, 33, 64)
    o, _, _ = oracle.compressed_attention(q, k_same, v)          # identical keys -> uniform weights
    assert max_abs(o, v.mean(dim=2, keepdim=True).expand_as(o)) < 1e-6
    k = torch.randn((1, 1, 33, 64), generator=g)
    perm = torch.randperm(33, generator=g)
    o1, _, _ = oracle.compressed_attention(q, k, v)
    o2, _, _ = oracle.compressed_attention(q, k[:, :, perm], v[:, :, perm])
    assert max_abs(o1, o2) < 1e-6                                # key permutation invariance


def test_compressed_fixture(golden):
    qc, kc, vc = (from_bf16_bits(golden[n]) for n in ("qc", "kc", "vc"))
    o, lse, s = oracle.compressed_attention(qc, kc, vc, out_dtype=torch.float32)
    assert max_abs(s, torch.from_numpy(golden["cmp_scores"])) < 2e-5
    assert max_abs(o, torch.from_numpy(golden["cmp_out"])) < 5e-6
    assert max_abs(lse, torch.from_numpy(golden["cmp_lse"])) < 5e-6


def test_flash_attn_topk_uses_unscaled_scores_and_model_order():
    g = torch.Generator().manual_seed(4)
    q, k, v = (torch.randn((1, 2, 100, 64), generator=g) for _ in range(3))
    o, idx = oracle.flash_attn_topk(q, k, v, 8)
    s = q @ k.transpose(-1, -2)
    want = torch.sort(s, dim=-1, descending=True, stable=True).indices[..., :8].to(torch.int32)
    assert torch.equal(idx, want)
    assert idx.dtype == torch.int32 and o.shape == q.shape


# ---------------------------------------------------------------- selection
def _rand_qkv(seed, h, n, d=64, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return tuple((torch.randn((1, h, n, d), generator=g) / (2.0 if i < 2 else 1.0)).to(dtype) for i in range(3))


@pytest.mark.parametrize("n,block,k", [(256, 64, 2), (200, 64, 3), (96, 16, 4), (100, 32, 2)])
def test_select_equals_dense_masked_brute_force(n, block, k):
    q, kk, v = _rand_qkv(10 + n, 2, n)
    nc = -(-n // block)
    g = torch.Generator().manual_seed(n)
    idx = torch.randint(-1, nc + 1, (1, 2, nc, k), generator=g, dtype=torch.int32)  # incl. -1 and out-of-range
    idx[..., 0] = torch.randint(0, nc, (1, 2, nc), generator=g, dtype=torch.int32)  # at least one valid entry
    got = oracle.select_attention(q, kk, v, idx, block)
    want = oracle.select_attention_dense_masked(q, kk, v, idx, block)
    assert max_abs(got, want) < 2e-6


def test_select_all_blocks_is_dense_attention():
    q, k, v = _rand_qkv(20, 2, 256)
    idx = torch.arange(4, dtype=torch.int32).view(1, 1, 1, 4).expand(1, 2, 4, 4).contiguous()
    assert max_abs(oracle.select_attention(q, k, v, idx, 64), F.scaled_dot_product_attention(q, k, v)) < 2e-6


def test_select_own_block_is_block_diagonal_and_duplicates_do_not_change_it():
    q, k, v = _rand_qkv(21, 1, 192)
    own = torch.arange(3, dtype=torch.int32).view(1, 1, 3, 1)
    got = oracle.select_attention(q, k, v, own, 64)
    for m in range(3):
        sl = slice(64 * m, 64 * (m + 1))
        want = F.scaled_dot_product_attention(q[:, :, sl], k[:, :, sl], v[:, :, sl])
        assert max_abs(got[:, :, sl], want) < 2e-6
    twice = own.expand(1, 1, 3, 2).contiguous()              # the same block twice: weights double, ratio unchanged
    assert max_abs(oracle.select_attention(q, k, v, twice, 64), got) < 2e-6


def test_select_duplicate_block_is_double_weighted():
    q, k, v = _rand_qkv(22, 1, 128)
    idx = torch.tensor([[[[0, 1, 1]], [[1, 0, 0]]]], dtype=torch.int32).view(1, 1, 2, 3)
    got = oracle.select_attention(q, k, v, idx, 64)
    s = (q[0, 0] @ k[0, 0].T) / 8.0
    w = torch.exp(s - s.max())
    w[:64, 64:] *= 2
    w[64:, :64] *= 2
    assert max_abs(got[0, 0], (w @ v[0, 0]) / w.sum(-1, keepdim=True)) < 2e-6


def test_select_skips_minus_one_and_empty_rows_give_zero():
    q, k, v = _rand_qkv(23, 1, 128)
    a = oracle.select_attention(q, k, v, torch.tensor([[[[1, -1], [0, 5]]]], dtype=torch.int32), 64)
    b = oracle.select_attention(q, k, v, torch.tensor([[[[1], [0]]]], dtype=torch.int32), 64)
    assert max_abs(a, b) == 0.0
    z = oracle.select_attention(q, k, v, torch.tensor([[[[-1], [0]]]], dtype=torch.int32), 64)
    assert torch.count_nonzero(z[:, :, :64]) == 0


def test_select_fixture(golden):
    q, k, v = (from_bf16_bits(golden[n]) for n in ("q", "k", "v"))
    idx = torch.from_numpy(golden["sel_idx"])
    got = oracle.select_attention(q, k, v, idx, 64, out_dtype=torch.float32)
    assert max_abs(got, torch.from_numpy(golden["sel_out"])) < 5e-6


# ---------------------------------------------------------------- merge and whole path
def test_merge_equals_reference_expression():
    g = torch.Generator().manual_seed(30)
    b, h, n, d, blk = 2, 3, 128, 8, 16
    o_sel = torch.randn((b, h, n, d), generator=g).to(torch.bfloat16)
    o_cmp = torch.randn((b, h, n // blk, d), generator=g).to(torch.bfloat16)
    gate = torch.sigmoid(torch.randn((b, h, n, 2), generator=g)).to(torch.bfloat16)
    # sparse_attention.py:127-136 written with plain view/broadcast ops
    sel_b = o_sel.view(b, h, n // blk, blk, d)
    gate_b = gate.view(b, h, n // blk, blk, 2)
    want = gate_b[..., 0:1] * o_cmp.view(b, h, n // blk, 1, d) + gate_b[..., 1:2] * sel_b
    want = want.permute(0, 2, 3, 1, 4).reshape(b, n, h * d)
    assert torch.equal(oracle.gated_merge(o_cmp, o_sel, gate, blk), want)


def test_merge_fixture_and_init_constants(golden):
    o_cmp, o_sel, gate, want = (from_bf16_bits(golden[n]) for n in ("merge_o_cmp", "merge_o_sel", "gate", "merge_out"))
    assert torch.equal(oracle.gated_merge(o_cmp, o_sel, gate, 64), want)
    g0, g1 = 1 / (1 + math.e), 1 / (1 + 1 / math.e)       # sigmoid(-1), sigmoid(+1): the reference's gate at init
    ones = torch.ones((1, 1, 64, 4))
    gate = torch.tensor([g0, g1]).view(1, 1, 1, 2).expand(1, 1, 64, 2)
    out = oracle.gated_merge(torch.full((1, 1, 1, 4), 2.0), ones, gate, 64)
    assert torch.allclose(out, torch.full((1, 64, 4), 2 * 0.26894142 + 0.73105858), atol=1e-6)


def test_whole_path_consistency():
    q, k, v = _rand_qkv(40, 2, 328)
    gate = torch.sigmoid(torch.randn((1, 2, 328, 2), generator=torch.Generator().manual_seed(41)))
    r = oracle.sparse_global_attention(q, k, v, gate, 64, 4)
    assert r["out"].shape == (1, 328, 128) and r["idx"].shape == (1, 2, 6, 4)
    # with K >= number of blocks every block is selected once -> selection equals dense attention
    r_all = oracle.sparse_global_attention(q, k, v, gate, 64, 8)
    pad_dup = r_all["idx"]                                    # 6 blocks, K=8: two filler slots repeat block 5
    assert (pad_dup[..., 6:] == 5).all()
    dense = F.scaled_dot_product_attention(q, k, v)
    s = (q @ k.transpose(-1, -2)) / 8.0
    w = torch.exp(s - s.amax(-1, keepdim=True))
    w[..., 320:] *= 3                                         # block 5 listed three times in total
    want = (w @ v) / w.sum(-1, keepdim=True)
    assert max_abs(r_all["o_sel"], want) < 2e-6
    assert max_abs(r_all["o_sel"], dense) > 1e-4              # and is measurably not plain dense attention
