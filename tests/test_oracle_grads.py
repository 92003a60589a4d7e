"""Pins of the backward oracle (CPU): the reference's formulas, torch autograd through the forward oracle, autograd
of the library attention and central differences must agree; the key-centric lists against plain loops."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from helpers import max_abs


def _randn(shape, seed, scale=1.0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float64) * scale).to(dtype)


def test_formula_equals_autograd_of_library_attention():
    q, k, v, g = (_randn((2, 3, 50, 16), s) for s in (1, 2, 3, 4))
    dq, dk, dv, o, lse = oracle.attention_grads_formula(q, k, v, g)
    qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))
    want = F.scaled_dot_product_attention(qq, kk, vv)
    want.backward(g)
    assert max_abs(o, want.detach()) <= 1e-12
    assert max_abs(dq, qq.grad) <= 1e-11 and max_abs(dk, kk.grad) <= 1e-11 and max_abs(dv, vv.grad) <= 1e-11
    # lse is the log of the softmax denominator of the scaled scores
    z = (q @ k.transpose(-1, -2)) / math.sqrt(16)
    assert max_abs(lse, torch.logsumexp(z, dim=-1)) <= 1e-12


def test_formula_matches_central_differences():
    q, k, v, g = (_randn((1, 1, 6, 4), s) for s in (5, 6, 7, 8))
    idx = torch.tensor([[[[0, 2], [1, 1], [-1, 0]]]], dtype=torch.int32)   # block 2: a duplicate and a skipped entry
    mult = oracle.block_multiplicity(idx, 6, 2)
    dq, dk, dv, _, _ = oracle.attention_grads_formula(q, k, v, g, mult)

    def loss(qq, kk, vv):
        return (oracle.select_attention_dense_masked(qq, kk, vv, idx, 2) * g).sum().item()

    eps = 1e-6
    for t, grad, which in ((q, dq, 0), (k, dk, 1), (v, dv, 2)):
        num = torch.zeros_like(t)
        for i in range(t.numel()):
            args = [q.clone(), k.clone(), v.clone()]
            args[which].view(-1)[i] += eps
            up = loss(*args)
            args[which].view(-1)[i] -= 2 * eps
            num.view(-1)[i] = (up - loss(*args)) / (2 * eps)
        assert max_abs(grad, num) <= 1e-7, which


def test_selection_autograd_paths_agree_with_the_formula():
    b, h, n, d, block, kk = 1, 2, 200, 8, 16, 3       # ragged: 200 = 12 * 16 + 8
    q, k, v, g = (_randn((b, h, n, d), s, 0.7) for s in (9, 10, 11, 12))
    gen = torch.Generator().manual_seed(13)
    nqb = -(-n // block)
    idx = torch.randint(-1, nqb + 1, (b, h, nqb, kk), generator=gen, dtype=torch.int32)   # includes -1 and out-of-range
    idx[0, 0, 3] = torch.tensor([5, 5, 2])                                                  # a duplicate
    mult = oracle.block_multiplicity(idx, n, block)
    dq, dk, dv, _, _ = oracle.attention_grads_formula(q, k, v, g, mult)
    bq, bk, bv = oracle.select_attention_grads_autograd(q, k, v, idx, block, g, brute_force=True)
    assert max_abs(dq, bq) <= 1e-10 and max_abs(dk, bk) <= 1e-10 and max_abs(dv, bv) <= 1e-10
    fq, fk, fv = oracle.select_attention_grads_autograd(q, k, v, idx, block, g)            # fp32 gather path
    assert max_abs(dq, fq) <= 2e-5 and max_abs(dk, fk) <= 2e-5 and max_abs(dv, fv) <= 2e-5


def test_compressed_autograd_agrees_with_the_formula():
    q, k, v, g = (_randn((2, 2, 70, 32), s, 0.5) for s in (14, 15, 16, 17))
    dq, dk, dv, _, _ = oracle.attention_grads_formula(q, k, v, g)
    aq, ak, av = oracle.compressed_attention_grads_autograd(q, k, v, g)
    assert max_abs(dq, aq) <= 2e-5 and max_abs(dk, ak) <= 2e-5 and max_abs(dv, av) <= 2e-5


def test_gradient_invariants():
    # dv rows of keys nobody attends are zero; the softmax rows sum to one, so adding a constant to all of v's rows
    # along the token axis leaves dq and dk unchanged
    q, k, v, g = (_randn((1, 1, 32, 8), s) for s in (18, 19, 20, 21))
    idx = torch.tensor([[[[0], [0]]]], dtype=torch.int32)          # block 16: key block 1 is never attended
    mult = oracle.block_multiplicity(idx, 32, 16)
    dq, dk, dv, _, _ = oracle.attention_grads_formula(q, k, v, g, mult)
    assert float(dv[0, 0, 16:].abs().max()) == 0.0 and float(dk[0, 0, 16:].abs().max()) == 0.0
    dq2, dk2, _, _, _ = oracle.attention_grads_formula(q, k, v + 3.0, g, mult)
    assert max_abs(dq, dq2) <= 1e-10 and max_abs(dk, dk2) <= 1e-10


def test_key_block_lists_of_the_oracle_hold_every_valid_entry_once_and_in_order():
    gen = torch.Generator().manual_seed(22)
    b, h, nqb, kk, nkb = 2, 3, 37, 4, 37
    idx = torch.randint(-2, nkb + 2, (b, h, nqb, kk), generator=gen, dtype=torch.int32)
    idx[1, 2, 5] = torch.tensor([7, 7, 7, 1])
    got = oracle.key_block_lists(idx, nkb)
    assert got[1 * h + 2][7].count(5) == 3 and got[1 * h + 2][1].count(5) == 1
    for bh in range(b * h):
        rows = idx.view(b * h, nqb, kk)[bh]
        assert sum(len(l) for l in got[bh]) == int(((rows >= 0) & (rows < nkb)).sum())
        for j in range(nkb):
            assert got[bh][j] == sorted(got[bh][j])
            for m in set(got[bh][j]):
                assert got[bh][j].count(m) == int((rows[m] == j).sum())


@pytest.mark.parametrize("name,block", [("b16", 16), ("b64", 64)])
def test_gradient_oracle_matches_the_brute_force_fixture(golden_grads, name, block):
    """The committed vectors come from an fp64 dense softmax under a multiplicity matrix, differentiated by autograd
    (tests/golden/make_grad_fixtures.py, independent of oracle/): both gradient routes of the oracle must reproduce
    them, duplicates, skipped and out-of-range entries, an empty row and the ragged last block included."""
    from helpers import from_bf16_bits

    q, k, v, g = (from_bf16_bits(golden_grads[n]) for n in ("q", "k", "v", "dout"))
    idx = torch.from_numpy(golden_grads[f"{name}_idx"])
    want = [torch.from_numpy(golden_grads[f"{name}_{t}"]) for t in ("dq", "dk", "dv")]
    got = oracle.select_attention_grads_autograd(q, k, v, idx, block, g)
    for a, w in zip(got, want):
        assert max_abs(a, w) <= 2e-5 * max(1.0, float(w.abs().max()))
    mult = oracle.block_multiplicity(idx, q.shape[2], block)
    dq, dk, dv, o, _ = oracle.attention_grads_formula(q, k, v, g, mult)
    for a, w in zip((dq, dk, dv), want):
        assert max_abs(a, w) <= 1e-6 * max(1.0, float(w.abs().max()))
    assert max_abs(torch.nan_to_num(o.float()), torch.from_numpy(golden_grads[f"{name}_out"])) <= 1e-6
