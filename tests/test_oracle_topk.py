"""Pins of the oracle's top-k model (CPU).

The reference has no tests; the order is fixed by its kernel text
(pi3/models/sparse_attn/flash_attention_topk.py:115-132,145-146, topk_utils.py:11-23).  These
tests pin the numpy model against: a tile-by-tile restatement of that text, a pure-Python
brute force (golden fixtures), stable torch.sort, and known answers for signed zeros, NaN
and ``K > Lk``.
"""
import numpy as np
import pytest
import torch

from oracle import sortable_key, topk_from_scores, topk_streaming


def test_sortable_key_known_values():
    x = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf], dtype=np.float32)
    k = sortable_key(x)
    assert k[0] == 0x80000000 and k[1] == 0x7FFFFFFF          # +0 above -0
    assert k[2] == (0x3F800000 | 0x80000000)
    assert k[3] == (~np.uint32(0xBF800000))
    assert k[4] > k[2] > k[0] > k[1] > k[3] > k[5]


def test_sortable_key_is_monotone():
    rng = np.random.default_rng(0)
    x = np.sort(rng.standard_normal(10000).astype(np.float32))
    k = sortable_key(x).astype(np.int64)
    assert np.all(np.diff(k) >= 0)
    assert np.all((np.diff(k) == 0) == (np.diff(x) == 0))


@pytest.mark.parametrize("name", ["smooth", "ties", "zeros", "short"])
def test_topk_matches_brute_force_fixture(golden, name):
    scores = golden[f"topk_{name}_scores"]
    want = golden[f"topk_{name}_idx"]
    got = topk_from_scores(scores, want.shape[1])
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("cols,k", [(64, 16), (65, 16), (131, 16), (300, 32), (1041, 8), (7, 16), (1, 4), (64, 64)])
def test_direct_model_equals_streaming_restatement(cols, k):
    rng = np.random.default_rng(cols * 100 + k)
    smooth = rng.standard_normal((9, cols)).astype(np.float32)
    ties = rng.integers(-2, 3, size=(9, cols)).astype(np.float32)
    for s in (smooth, ties):
        np.testing.assert_array_equal(topk_from_scores(s, k), topk_streaming(s, k))


def test_matches_stable_torch_sort_without_signed_zero_mixes():
    g = torch.Generator().manual_seed(3)
    s = torch.randint(-4, 5, (32, 500), generator=g).float()
    s[s == 0] = 0.5  # keep +-0 out: torch orders -0 == +0, the reference orders +0 first
    want = torch.sort(s, dim=-1, descending=True, stable=True).indices[:, :16].to(torch.int32).numpy()
    np.testing.assert_array_equal(topk_from_scores(s, 16), want)


def test_signed_zero_and_nan_known_answers():
    s = np.full((1, 8), -1.0, dtype=np.float32)
    s[0, 5] = -0.0
    s[0, 6] = 0.0
    np.testing.assert_array_equal(topk_from_scores(s, 2), [[6, 5]])
    s = np.array([[1.0, np.inf, np.nan, 2.0]], dtype=np.float32)   # positive quiet NaN ranks above +inf
    assert np.signbit(s[0, 2]) == False  # noqa: E712
    np.testing.assert_array_equal(topk_from_scores(s, 4), [[2, 1, 3, 0]])


def test_fewer_columns_than_k_fills_with_last_column():
    s = np.array([[3.0, 1.0, 2.0]], dtype=np.float32)
    np.testing.assert_array_equal(topk_from_scores(s, 8), [[0, 2, 1, 2, 2, 2, 2, 2]])
    np.testing.assert_array_equal(topk_streaming(s, 8), [[0, 2, 1, 2, 2, 2, 2, 2]])


def test_invariants_unique_sorted_and_permutation_equivariant():
    rng = np.random.default_rng(11)
    s = rng.standard_normal((16, 777)).astype(np.float32)
    idx = topk_from_scores(s, 16)
    assert all(len(set(r)) == 16 for r in idx.tolist())
    picked = np.take_along_axis(s, idx.astype(np.int64), axis=1)
    assert np.all(np.diff(picked, axis=1) <= 0)
    assert np.all(picked[:, -1:] >= np.sort(s, axis=1)[:, -16:-15])
    perm = rng.permutation(777)
    idx_p = topk_from_scores(s[:, perm], 16)          # tie-free data: selecting commutes with permuting columns
    np.testing.assert_array_equal(perm[idx_p], idx)
