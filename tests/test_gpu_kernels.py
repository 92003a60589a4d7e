"""Parity of each HIP kernel against the CPU oracle, through the C-ABI (needs an MI355X).

Bars: integer/index results bit-exact; floating point within 2e-2 max-abs for bf16/fp16 I/O and
1e-5 for fp32 I/O of the oracle evaluated in fp32 on the same (already rounded) inputs.
"""
import numpy as np
import pytest
import torch

import oracle
import speed3r_amd as s3r
from helpers import from_bf16_bits, max_abs, merged_within_rounding

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 2e-2}


def _randn(shape, seed, dtype, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def _ulp_close(got, want_f32, dtype):
    """|got - want| within one rounding step of dtype (want given in fp32)."""
    rel = {torch.float32: 2e-6, torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -10}[dtype]
    err = (got.float().cpu() - want_f32).abs()
    return bool((err <= rel * want_f32.abs() + 1e-6).all())


# ------------------------------------------------------------------------------------ pooling
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("n,block,d", [(256, 64, 64), (200, 64, 64), (1041, 64, 64), (96, 16, 64), (130, 32, 32), (7, 64, 64),
                                       (1041, 16, 64), (1000, 8, 64), (333, 32, 64), (5, 16, 64), (64, 16, 64), (200, 4, 64)])
def test_pool_matches_oracle(dtype, n, block, d):
    x = _randn((2, 3, n, d), n + d, dtype)
    got = s3r.pool_mean(x.to(DEV), block)
    assert got.shape == (2, 3, -(-n // block), d) and got.dtype == dtype
    assert _ulp_close(got, oracle.pool_mean(x, block, out_dtype=torch.float32), dtype)


def test_pool_fixture_and_packed_qkv_view(golden):
    H, N, D = 2, 200, 64
    q, k, v = (from_bf16_bits(golden[n]) for n in ("q", "k", "v"))
    for name, t in (("q", q), ("k", k), ("v", v)):
        got = s3r.pool_mean(t.to(DEV), 64)
        assert _ulp_close(got, torch.from_numpy(golden[f"pooled_{name}"]), torch.bfloat16)
    # the layer's packed projection [B, N, (qkv h d)] pooled in one launch through strides
    packed = torch.stack([q, k, v], dim=0)[:, 0].permute(2, 0, 1, 3).reshape(1, N, 3 * H * D).contiguous()
    qc, kc, vc = s3r.pool_qkv_packed(packed.to(DEV), H, 64)
    for name, got in (("q", qc), ("k", kc), ("v", vc)):
        assert _ulp_close(got, torch.from_numpy(golden[f"pooled_{name}"]), torch.bfloat16)


# ------------------------------------------------------------------------------------ merge
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("n,block", [(256, 64), (200, 64), (96, 16)])
def test_merge_bit_exact(dtype, n, block):
    b, h, d = 2, 4, 64
    o_sel = _randn((b, h, n, d), 1, dtype)
    o_cmp = _randn((b, h, -(-n // block), d), 2, dtype)
    gate_lin = torch.sigmoid(_randn((b, n, 2 * h), 3, torch.float32)).to(dtype)
    gate = gate_lin.view(b, n, h, 2).permute(0, 2, 1, 3)          # the reference's strided 'b n (h g) -> b h n g' view
    got = s3r.gated_merge(o_cmp.to(DEV), o_sel.to(DEV), gate_lin.to(DEV).view(b, n, h, 2).permute(0, 2, 1, 3), block)
    want = oracle.gated_merge(o_cmp, o_sel, gate, block)
    assert got.shape == (b, n, h * d)
    assert torch.equal(got.cpu(), want)


def test_merge_fixture(golden):
    o_cmp, o_sel, gate, want = (from_bf16_bits(golden[n]) for n in ("merge_o_cmp", "merge_o_sel", "gate", "merge_out"))
    got = s3r.gated_merge(o_cmp.to(DEV), o_sel.to(DEV), gate.to(DEV), 64)
    assert torch.equal(got.cpu(), want)


# ------------------------------------------------------------------------------------ top-k
@pytest.mark.parametrize("name", ["smooth", "ties", "zeros", "short"])
def test_topk_fixture_bit_exact(golden, name):
    scores = torch.from_numpy(golden[f"topk_{name}_scores"])
    want = golden[f"topk_{name}_idx"]
    got = s3r.topk_rows(scores.to(DEV), want.shape[1])
    np.testing.assert_array_equal(got.cpu().numpy(), want)


@pytest.mark.parametrize("cols", [1, 5, 63, 64, 65, 131, 1041, 4164])
@pytest.mark.parametrize("k", [1, 8, 16, 32, 64])
def test_topk_random_and_tie_heavy_bit_exact(cols, k):
    rng = np.random.default_rng(cols * 131 + k)
    smooth = rng.standard_normal((37, cols)).astype(np.float32)
    ties = rng.integers(-2, 3, size=(37, cols)).astype(np.float32)
    ties[ties == 0] = np.where(rng.random(np.count_nonzero(ties == 0)) < 0.5, 0.0, -0.0)   # signed zeros mixed in
    for s in (smooth, ties):
        got = s3r.topk_rows(torch.from_numpy(s).to(DEV), k).cpu().numpy()
        np.testing.assert_array_equal(got, oracle.topk_from_scores(s, k))


def test_topk_special_values_bit_exact():
    s = np.array([[1.0, np.inf, np.nan, 2.0, -np.inf, -0.0, 0.0, -np.nan]], dtype=np.float32)
    got = s3r.topk_rows(torch.from_numpy(s).to(DEV), 8).cpu().numpy()
    np.testing.assert_array_equal(got, oracle.topk_from_scores(s, 8))


# ------------------------------------------------------------------------------------ compressed branch
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("lq,lk", [(150, 150), (131, 131), (64, 64), (1, 1), (100, 300), (300, 100), (1041, 1041)])
def test_compressed_matches_oracle(dtype, lq, lk):
    h, d, k = 3, 64, 16
    q = _randn((1, h, lq, d), lq, dtype, 0.5)
    kk = _randn((1, h, lk, d), lk + 1, dtype, 0.5)
    v = _randn((1, h, lk, d), lk + 2, dtype)
    o, idx, scores, lse = s3r.compressed_attn_topk(q.to(DEV), kk.to(DEV), v.to(DEV), k, return_scores=True, return_lse=True)
    o_ref, lse_ref, s_ref = oracle.compressed_attention(q, kk, v, out_dtype=torch.float32)
    assert max_abs(o, o_ref) <= TOL[dtype]
    assert max_abs(lse, lse_ref) <= (1e-4 if dtype == torch.float32 else 2e-3)  # 16-bit: row sums are over rounded probabilities
    assert max_abs(scores, s_ref) <= 1e-4                           # same products, different summation order
    # indices are exact for the scores the kernel produced
    np.testing.assert_array_equal(idx.cpu().numpy(), oracle.topk_from_scores(scores.cpu(), k))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("h,n", [(3, 1), (3, 63), (2, 64), (3, 65), (2, 128), (3, 129), (2, 200), (3, 1041), (16, 4164), (24, 4096), (33, 4000)])
def test_dense_sweep_of_the_pipelined_kernel_matches_oracle(dtype, h, n):
    """The attention of the compressed branch without a score buffer runs as a dense sweep of the selection kernel:
    with few query blocks two waves share a block and sweep half of the key tiles each (every case here but the
    last two), otherwise one wave sweeps them all (24 heads x 64 blocks) -- unless the waves fill the chip a whole
    number of times plus a small rest, which again takes two waves per block (33 heads x 63 blocks = 2048 + 31).  One
    to 66 tiles, ragged last tiles, odd and even tile counts, a last workgroup with a single pair."""
    q = _randn((1, h, n, 64), n, dtype, 0.5)
    k = _randn((1, h, n, 64), n + 1, dtype, 0.5)
    v = _randn((1, h, n, 64), n + 2, dtype)
    o, idx, lse = s3r.compressed_attn_topk(q.to(DEV), k.to(DEV), v.to(DEV), None, return_lse=True)
    assert idx is None
    o_ref, lse_ref, _ = oracle.compressed_attention(q, k, v, out_dtype=torch.float32)
    assert max_abs(o, o_ref) <= TOL[dtype]
    assert max_abs(lse, lse_ref) <= 2e-3


def test_compressed_fixture(golden):
    qc, kc, vc = (from_bf16_bits(golden[n]) for n in ("qc", "kc", "vc"))
    o, idx, scores = s3r.compressed_attn_topk(qc.to(DEV), kc.to(DEV), vc.to(DEV), 8, return_scores=True)
    assert max_abs(o, torch.from_numpy(golden["cmp_out"])) <= 2e-2
    assert max_abs(scores, torch.from_numpy(golden["cmp_scores"])) <= 1e-4


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("k", [1, 2, 4, 8, 16, 32])
@pytest.mark.parametrize("lq,lk", [(150, 150), (64, 64), (5, 5), (100, 300), (300, 100), (1041, 1041), (130, 4164)])
def test_fused_selection_equals_selection_from_stored_scores(dtype, k, lq, lk):
    """The fused top-k never sees HBM scores; the same kernel with a score buffer produces bit-identical
    scores, so both index sets must agree bit for bit with the oracle's order on those scores."""
    h = 2
    q = _randn((1, h, lq, 64), lq + k, dtype, 0.5).to(DEV)
    kk = _randn((1, h, lk, 64), lk + 1, dtype, 0.5)
    kk[:, :, lk // 2:] = kk[:, :, :lk - lk // 2]          # duplicated keys: exact score ties, lowest column must win
    kk = kk.to(DEV)
    v = _randn((1, h, lk, 64), lk + 2, dtype).to(DEV)
    o_f, idx_f = s3r.compressed_attn_topk(q, kk, v, k, materialize_scores=False)
    o_m, idx_m, scores = s3r.compressed_attn_topk(q, kk, v, k, return_scores=True)
    want = oracle.topk_from_scores(scores.cpu(), k)
    np.testing.assert_array_equal(idx_m.cpu().numpy(), want)
    np.testing.assert_array_equal(idx_f.cpu().numpy(), want)
    # the two routes compute the attention output with different kernels (dense sweep of the selection kernel vs the
    # score-writing kernel): same mathematics, different summation order
    assert max_abs(o_f, o_m.float()) <= 2e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("k", [1, 8, 16, 32])
@pytest.mark.parametrize("h,lq,lk", [(26, 2000, 300), (16, 4164, 1041), (13, 4100, 65)])
def test_fused_selection_in_two_wave_workgroups(dtype, k, h, lq, lk):
    """Between 768 and 1280 (64-row block, head) pairs the index kernel runs workgroups of two waves (a ring of two K
    tiles, four transfer instructions per wave and tile): the same bit-exact agreement with the oracle's order on the
    stored scores, ties included, ragged last query block and ragged last key tile."""
    pairs = -(-lq // 64) * h
    assert 768 < pairs <= 1280
    q = _randn((1, h, lq, 64), lq + k, dtype, 0.5).to(DEV)
    kk = _randn((1, h, lk, 64), lk + 1, dtype, 0.5)
    kk[:, :, lk // 2:] = kk[:, :, :lk - lk // 2]          # duplicated keys: exact score ties, lowest column must win
    kk = kk.to(DEV)
    _, idx_f = s3r.compressed_attn_topk(q, kk, None, k, materialize_scores=False)
    v = _randn((1, h, lk, 64), lk + 2, dtype).to(DEV)
    _, idx_m, scores = s3r.compressed_attn_topk(q, kk, v, k, return_scores=True)
    want = oracle.topk_from_scores(scores.cpu(), k)
    np.testing.assert_array_equal(idx_m.cpu().numpy(), want)
    np.testing.assert_array_equal(idx_f.cpu().numpy(), want)


def test_fused_selection_special_scores():
    """Zero queries give all-zero scores (every column ties: indices 0..K-1); a huge key gives +inf scores."""
    lk = 200
    q = torch.zeros((1, 1, 70, 64), dtype=torch.bfloat16, device=DEV)
    kk = _randn((1, 1, lk, 64), 3, torch.bfloat16).to(DEV)
    v = _randn((1, 1, lk, 64), 4, torch.bfloat16).to(DEV)
    _, idx = s3r.compressed_attn_topk(q, kk, v, 16, materialize_scores=False)
    assert torch.equal(idx.cpu(), torch.arange(16, dtype=torch.int32).expand(1, 1, 70, 16))
    q = _randn((1, 1, 70, 64), 5, torch.bfloat16).to(DEV)
    kk[0, 0, 150] = 3e38
    _, idx_f = s3r.compressed_attn_topk(q, kk, v, 8, materialize_scores=False)
    _, idx_m, scores = s3r.compressed_attn_topk(q, kk, v, 8, return_scores=True)
    np.testing.assert_array_equal(idx_f.cpu().numpy(), oracle.topk_from_scores(scores.cpu(), 8))


def test_flash_attn_topk_func_signature():
    q = _randn((1, 2, 200, 64), 5, torch.bfloat16, 0.5)
    o, idx = s3r.flash_attn_topk_func(q.to(DEV), q.to(DEV), q.to(DEV), 16)
    assert o.shape == q.shape and o.dtype == q.dtype
    assert idx.shape == (1, 2, 200, 16) and idx.dtype == torch.int32
    assert (idx[..., 0].cpu() == torch.arange(200)).float().mean() > 0.95     # q.q is (almost always) the row maximum
    # bias is accepted and ignored, as in the reference (flash_attention_topk.py:646-648)
    o2, idx2 = s3r.flash_attn_topk_func(q.to(DEV), q.to(DEV), q.to(DEV), 16, torch.ones((1, 2, 200, 200), device=DEV))
    assert torch.equal(o2, o) and torch.equal(idx2, idx)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("lq,lk,k", [(150, 150, 16), (200, 200, 64), (100, 180, 8), (130, 70, 32), (40, 40, 64), (3, 2, 4), (1041, 1041, 16)])
def test_causal_variant_matches_oracle(dtype, lq, lk, k):
    """flash_attn_topk_func(causal=True), the reference kernel's IS_CAUSAL branches: attention within the dtype's
    tolerance (1e-5 fp32, 2e-2 bf16/fp16), indices bit for bit from the scores the kernel stored, and those scores
    against the oracle's (fp32 products in another order: 1e-4 of the largest score)."""
    h = 2
    q = _randn((1, h, lq, 64), 21, dtype, 0.5)
    kk = _randn((1, h, lk, 64), 22, dtype, 0.5)
    v = _randn((1, h, lk, 64), 23, dtype, 1.0)
    o, idx, scores, lse = s3r.compressed_attn_topk(q.to(DEV), kk.to(DEV), v.to(DEV), k, causal=True, return_scores=True, return_lse=True)
    want_o, want_lse, want_s = oracle.compressed_attention(q, kk, v, p_dtype=None if dtype == torch.float32 else dtype,
                                                           out_dtype=torch.float32, causal=True)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert max_abs(o, want_o) <= tol
    assert (lse.cpu() - want_lse).abs().max().item() <= 1e-4
    sc = scores.cpu()
    for m0 in range(0, lq, 64):
        end_n = min(m0 + 64, lk)
        got, want = sc[:, :, m0:m0 + 64, :end_n], want_s[:, :, m0:m0 + 64, :end_n]
        assert torch.equal(torch.isinf(got), torch.isinf(want))
        fin = torch.isfinite(want)
        assert (got[fin] - want[fin]).abs().max().item() <= 1e-4 * max(1.0, want[fin].abs().max().item())
        assert torch.isnan(sc[:, :, m0:m0 + 64, end_n:]).all()          # columns the block does not visit stay untouched
    from oracle import sparse_attention_oracle as so
    np.testing.assert_array_equal(idx.cpu().numpy(), so.topk_from_scores_causal(sc, k))
    o2, idx2 = s3r.flash_attn_topk_func(q.to(DEV), kk.to(DEV), v.to(DEV), k, None, True)
    assert torch.equal(o2, o) and torch.equal(idx2, idx)


def test_causal_variant_backward_is_the_non_causal_backward_on_the_causal_lse():
    """The reference's backward does not know of `causal` (flash_attention_topk.py:653-666): dq, dk, dv are those of
    the dense operator evaluated with the forward's (causal) log-sum-exp and output."""
    from speed3r_amd.sparse_attn import ops
    lq = 200
    q, kk, v = (_randn((1, 2, lq, 64), s, torch.bfloat16, 0.5).to(DEV).requires_grad_(True) for s in (31, 32, 33))
    o, _ = s3r.flash_attn_topk_func(q, kk, v, 8, None, True)
    g = _randn((1, 2, lq, 64), 34, torch.bfloat16, 1.0).to(DEV)
    o.backward(g)
    with torch.no_grad():
        o_c, _, lse_c = ops.compressed_attn_topk(q, kk, v, 8, causal=True, return_lse=True)
        dq, dk, dv = ops.attn_bwd(q, kk, v, o_c, g, lse_c, None, 64, None)
    assert torch.equal(q.grad, dq) and torch.equal(kk.grad, dk) and torch.equal(v.grad, dv)


# ------------------------------------------------------------------------------------ selection branch
def _rand_idx(h, nc, k, seed, with_invalid=True):
    g = torch.Generator().manual_seed(seed)
    lo, hi = (-1, nc + 1) if with_invalid else (0, nc)
    idx = torch.randint(lo, hi, (1, h, nc, k), generator=g, dtype=torch.int32)
    idx[..., 0] = torch.randint(0, nc, (1, h, nc), generator=g, dtype=torch.int32)
    return idx


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("n,block,k", [(256, 64, 4), (200, 64, 3), (1041, 64, 16), (2112, 64, 8), (96, 16, 4), (100, 32, 2), (40, 4, 3)])
def test_select_matches_oracle(dtype, n, block, k):
    h = 3
    q = _randn((1, h, n, 64), n, dtype, 0.5)
    kk = _randn((1, h, n, 64), n + 1, dtype, 0.5)
    v = _randn((1, h, n, 64), n + 2, dtype)
    idx = _rand_idx(h, -(-n // block), k, n)
    o, lse = s3r.select_attn(q.to(DEV), kk.to(DEV), v.to(DEV), idx.to(DEV), block, return_lse=True)
    o_ref, lse_ref = oracle.select_attention(q, kk, v, idx, block, out_dtype=torch.float32, return_lse=True)
    assert o.dtype == dtype and o.shape == q.shape
    assert max_abs(o, o_ref) <= TOL[dtype]
    assert max_abs(lse, lse_ref) <= (1e-4 if dtype == torch.float32 else 2e-3)  # 16-bit: row sums are over rounded probabilities


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,k,with_invalid", [(96, 4, False), (1041, 32, False), (1041, 32, True), (200, 7, True), (16, 1, False),
                                              (2000, 64, True), (70, 3, True)])
def test_select_block16_matches_oracle(dtype, n, k, with_invalid):
    """16-token blocks (the reference layer's own setting) on their MFMA kernel (a wave walks the union of four query
    blocks' lists): ragged lengths, group tails (query-block counts that are not multiples of four), skipped and
    duplicated entries."""
    h, block = 2, 16
    nqb = -(-n // block)
    q = _randn((1, h, n, 64), n, dtype, 0.5)
    kk = _randn((1, h, n, 64), n + 1, dtype, 0.5)
    v = _randn((1, h, n, 64), n + 2, dtype)
    g = torch.Generator().manual_seed(n + k)
    lo, hi = (-1, nqb + 1) if with_invalid else (0, nqb)
    idx = torch.randint(lo, hi, (1, h, nqb, k), generator=g, dtype=torch.int32)
    if with_invalid:
        idx[0, 0, 0, :] = -1                    # a query block that attends nothing
        if k > 1:
            idx[0, 1, nqb - 1, 1] = idx[0, 1, nqb - 1, 0]   # a duplicate
    o, lse = s3r.select_attn(q.to(DEV), kk.to(DEV), v.to(DEV), idx.to(DEV), block, return_lse=True)
    o_ref, lse_ref = oracle.select_attention(q, kk, v, idx, block, out_dtype=torch.float32, return_lse=True)
    assert o.dtype == dtype and o.shape == q.shape
    assert max_abs(o, o_ref) <= TOL[dtype]
    fin = torch.isfinite(lse_ref)
    assert torch.equal(torch.isfinite(lse.cpu()), fin)
    assert max_abs(lse.cpu()[fin], lse_ref[fin]) <= 2e-3
    if with_invalid:
        assert float(o[0, 0, :16].float().abs().max()) == 0.0


def test_select_fixture(golden):
    q, k, v = (from_bf16_bits(golden[n]) for n in ("q", "k", "v"))
    idx = torch.from_numpy(golden["sel_idx"])
    o = s3r.topk_blocksparse_attention(q.to(DEV), k.to(DEV), v.to(DEV), idx.to(DEV), 64)
    assert max_abs(o, torch.from_numpy(golden["sel_out"])) <= 2e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,h,kk,block", [(256, 2, 2, 64), (200, 3, 4, 64), (1041, 2, 16, 64), (64, 1, 1, 64),
                                          (256, 2, 4, 16), (200, 3, 8, 16), (1041, 2, 32, 16), (40, 1, 1, 16)])
def test_select_with_fused_merge_equals_the_two_operators(dtype, n, h, kk, block):
    """The merge in the selection kernel's epilogue against select_attn followed by gated_merge (ragged tail, skipped
    entries and empty rows included) and against the oracle's merge of the oracle's selection.  The 16-token kernel
    rounds like the eager expression (selection output, both products, sum): the same bits.  The 64-token kernel
    evaluates gate0 * o_cmp + gate1 * o_sel in fp32 and rounds once: within the rounding steps between the two."""
    b, d = 2, 64
    nqb = -(-n // block)
    q, k, v = (_randn((b, h, n, d), 20 + i, dtype, 0.5).to(DEV) for i in range(3))
    g = torch.Generator().manual_seed(5)
    idx = torch.randint(-1, nqb + 1, (b, h, nqb, kk), generator=g, dtype=torch.int32)   # -1 and nqb are skipped entries
    idx[0, 0, 0, :] = -1                                                                  # an empty row
    o_cmp = _randn((b, h, nqb, d), 30, dtype).to(DEV)
    gate_lin = torch.sigmoid(_randn((b, n, 2 * h), 31, torch.float32)).to(dtype).to(DEV)
    gate = gate_lin.view(b, n, h, 2).permute(0, 2, 1, 3)                                  # strided view, contiguous pair
    o_sel = s3r.select_attn(q, k, v, idx.to(DEV), block)
    want = s3r.gated_merge(o_cmp, o_sel, gate, block)
    got = s3r.select_attn_merge(q, k, v, idx.to(DEV), o_cmp, gate, block)
    assert got is not None and got.shape == (b, n, h * d)
    if block == 16:
        assert torch.equal(got, want)
    else:
        assert merged_within_rounding(got, o_cmp, o_sel, gate, block)
        empty = o_sel[0, 0, :block].float().abs().max() == 0                          # the empty row merges zeros
        assert empty and merged_within_rounding(got[:1, :block, :d], o_cmp[:1, :1], o_sel[:1, :1, :block], gate[:1, :1, :block], block)
    ref_sel = oracle.select_attention(q.cpu(), k.cpu(), v.cpu(), idx, block, out_dtype=torch.float32)
    ref = oracle.gated_merge(o_cmp.cpu().float(), ref_sel, gate.cpu().float(), block)
    assert max_abs(got, ref) <= 3e-2


def test_fused_merge_declines_shapes_without_an_mfma_kernel():
    b, h, n, d, block = 1, 2, 96, 64, 32
    q, k, v = (_randn((b, h, n, d), 40 + i, torch.bfloat16).to(DEV) for i in range(3))
    idx = torch.zeros((b, h, n // block, 2), dtype=torch.int32, device=DEV)
    o_cmp = _randn((b, h, n // block, d), 43, torch.bfloat16).to(DEV)
    gate = torch.rand((b, h, n, 2), dtype=torch.float32).to(torch.bfloat16).to(DEV)
    assert s3r.select_attn_merge(q, k, v, idx, o_cmp, gate, block) is None
    out = s3r.sparse_global_attention(q, k, v, gate, block=block, topk=2)      # falls back to the two operators
    assert out.shape == (b, n, h * d)


def test_select_empty_row_gives_zeros_and_strided_inputs_work():
    n, h = 256, 2
    qkv = _randn((1, n, 3, h, 64), 9, torch.bfloat16, 0.5).to(DEV)
    q, k, v = (qkv[:, :, i].transpose(1, 2) for i in range(3))        # [1,h,n,64] strided views of a packed buffer
    idx = torch.tensor([[-1, -1], [0, 1], [2, 2], [3, 9]], dtype=torch.int32).view(1, 1, 4, 2).expand(1, h, 4, 2).contiguous()
    o = s3r.select_attn(q, k, v, idx.to(DEV), 64)
    assert torch.count_nonzero(o[:, :, :64]) == 0
    o_ref = oracle.select_attention(q.cpu(), k.cpu(), v.cpu(), idx, 64, out_dtype=torch.float32)
    assert max_abs(o, o_ref) <= 2e-2


def test_select_handles_scores_far_above_the_first_tile():
    """The MFMA kernel takes the first half tile's row maximum as the softmax reference; when later tiles exceed it by
    more than fp32 can hold it must fall back to the online softmax.  Block 0 listed first has tiny scores,
    block 2 has logits around +140 in base-2 units above them (exp2 overflows fp32)."""
    g = torch.Generator().manual_seed(5)
    n = 256
    q = (torch.randn((1, 2, n, 64), generator=g)).to(torch.bfloat16)
    k = (torch.randn((1, 2, n, 64), generator=g) * 0.01).to(torch.bfloat16)
    k[:, :, 128:192] = (q[:, :, 0:64] * 12.0)          # block 2: logits ~140 (base 2) above block 0's
    v = torch.randn((1, 2, n, 64), generator=g).to(torch.bfloat16)
    idx = torch.tensor([[0, 2, 1], [1, 0, 3], [2, 3, 0], [3, 1, 2]], dtype=torch.int32).view(1, 1, 4, 3).expand(1, 2, 4, 3).contiguous()
    o = s3r.select_attn(q.to(DEV), k.to(DEV), v.to(DEV), idx.to(DEV), 64)
    ref = oracle.select_attention(q, k, v, idx, 64, out_dtype=torch.float32)
    assert torch.isfinite(o.float()).all() and max_abs(o, ref) <= 2e-2


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("gain", [2.0, 2.5])
def test_select_fp16_probabilities_above_the_first_half_tile_stay_finite(dtype, gain):
    """The 64-token kernel never rescales: a probability is exp2(score - row maximum of the FIRST half tile).  A later
    block 14..40 base-2 units above that reference gives probabilities up to 2^40: fine in bf16, beyond fp16's 65504,
    where the rounded probability would be inf while the fp32 row sum stays far below the 2^100 that triggers the
    fallback for bf16.  The running-max softmax of the reference kernel (topk_blocksparse_attention.py:104-119) cannot
    overflow, so neither may this: list instance, fused-merge instance and dense sweep (one and two waves per query
    block), against the oracle."""
    g = torch.Generator().manual_seed(5)
    n, h = 256, 2
    q = torch.randn((1, h, n, 64), generator=g).to(dtype)
    k = (torch.randn((1, h, n, 64), generator=g) * 0.01).to(dtype)
    k[:, :, 128:192] = (q[:, :, 0:64] * gain).to(dtype)     # block 2: row i of block 0 scores |q_i|^2 * gain / 8 on key 128 + i
    v = torch.randn((1, h, n, 64), generator=g).to(dtype)
    planted = (q[:, :, 0:64].float() * k[:, :, 128:192].float()).sum(-1) * 0.125 * 1.4426950408889634
    assert planted.min() > 10 and planted.max() > 24             # base-2 units above the (tiny) scores of the other blocks
    idx = torch.tensor([[0, 2, 1], [1, 0, 3], [2, 3, 0], [3, 1, 2]], dtype=torch.int32).view(1, 1, 4, 3).expand(1, h, 4, 3).contiguous()
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    ref = oracle.select_attention(q, k, v, idx, 64, out_dtype=torch.float32)
    o = s3r.select_attn(qd, kd, vd, idx.to(DEV), 64)
    assert torch.isfinite(o.float()).all() and max_abs(o, ref) <= 2e-2
    # merge in the epilogue
    o_cmp = _randn((1, h, 4, 64), 30, dtype)
    gate = torch.sigmoid(_randn((1, h, n, 2), 31, torch.float32)).to(dtype)
    got = s3r.select_attn_merge(qd, kd, vd, idx.to(DEV), o_cmp.to(DEV), gate.to(DEV), 64)
    want = oracle.gated_merge(o_cmp.float(), ref, gate.float(), 64)
    assert torch.isfinite(got.float()).all() and max_abs(got, want) <= 3e-2
    # dense sweep, two waves per query block: the second wave of block 0 starts at tile 2, whose second half holds the
    # planted keys of rows 32..63
    od, none, lse = s3r.compressed_attn_topk(qd, kd, vd, None, return_lse=True)
    o_ref, lse_ref, _ = oracle.compressed_attention(q, k, v, out_dtype=torch.float32)
    assert none is None and torch.isfinite(od.float()).all() and max_abs(od, o_ref) <= 2e-2
    # the log-sum-exp is about the planted score here (10 to 30 nats): the queries carry the softmax scale rounded to the
    # I/O type, 2^-9 (bf16) of every product q_d k_d, which all have one sign for the planted key
    assert ((lse.cpu() - lse_ref).abs() <= 2e-3 + 5e-4 * lse_ref.abs()).all()


def test_dense_sweep_fp16_probabilities_above_the_first_half_tile_one_wave_per_block():
    """Same hole in the dense sweep with one wave per query block (24 heads x 64 blocks): the planted keys sit 32
    tiles after the tile that fixed the reference."""
    g = torch.Generator().manual_seed(6)
    n, h = 4096, 24
    q = torch.randn((1, h, n, 64), generator=g).to(torch.float16)
    k = (torch.randn((1, h, n, 64), generator=g) * 0.01).to(torch.float16)
    k[:, :, 2048:2112] = (q[:, :, 0:64] * 2.0).to(torch.float16)
    v = torch.randn((1, h, n, 64), generator=g).to(torch.float16)
    od, _ = s3r.compressed_attn_topk(q.to(DEV), k.to(DEV), v.to(DEV), None)
    o_ref, _, _ = oracle.compressed_attention(q, k, v, out_dtype=torch.float32)
    assert torch.isfinite(od.float()).all() and max_abs(od, o_ref) <= 2e-2


def test_forward_only_guard():
    x = torch.zeros((1, 1, 64, 64), dtype=torch.bfloat16, device=DEV, requires_grad=True)
    with pytest.raises(RuntimeError, match="forward-only"):
        s3r.pool_mean(x, 64)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("rows,c", [(1, 8), (7, 1024), (1030, 1024), (5, 136), (3, 2048), (9, 512)])
def test_layer_norm_matches_fp64_closed_form(dtype, rows, c):
    """s3r_layer_norm against (x - mean) / sqrt(var + eps) * w + b evaluated in fp64 on the same inputs; the result is
    rounded once to the I/O dtype: half an ulp of the output plus the fp32 error of the statistics."""
    from speed3r_amd.sparse_attn import ops
    g = torch.Generator().manual_seed(rows * 131 + c)
    x = (torch.randn(rows, c, generator=g) * 3 + 0.5).to(dtype).to("cuda:0")
    w = (torch.randn(c, generator=g)).to(dtype).to("cuda:0")
    b = (torch.randn(c, generator=g)).to(dtype).to("cuda:0")
    for bias in (b, None):
        got = ops.layer_norm(x, w, bias, 1e-6)
        assert got is not None and got.shape == x.shape and got.dtype == dtype
        xd = x.double()
        mean = xd.mean(-1, keepdim=True)
        var = ((xd - mean) ** 2).mean(-1, keepdim=True)
        ref = (xd - mean) / torch.sqrt(var + 1e-6) * w.double() + (bias.double() if bias is not None else 0.0)
        ulp = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -22}[dtype]
        assert ((got.double() - ref).abs() <= ulp * ref.abs() + 1e-5).all()
    # constant rows: zero variance, the output is the bias
    xc = torch.full((4, c), 2.5, dtype=dtype, device="cuda:0")
    assert torch.equal(ops.layer_norm(xc, w, b, 1e-6), b.expand(4, c))


def test_layer_norm_declines_rows_it_has_no_kernel_for():
    from speed3r_amd.sparse_attn import ops
    w = torch.ones(12, dtype=torch.bfloat16, device="cuda:0")
    assert ops.layer_norm(torch.ones(3, 12, dtype=torch.bfloat16, device="cuda:0"), w, None, 1e-6) is None


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("n,block,k,with_invalid", [(512, 128, 2, False), (1041, 128, 4, True), (1041, 256, 3, True),
                                                    (2000, 256, 8, False), (100, 128, 1, False), (300, 256, 2, True)])
def test_select_blocks_of_128_and_256_tokens_match_oracle(dtype, n, block, k, with_invalid):
    """The reference operator also takes blocks of 128 and 256 tokens (topk_blocksparse_attention.py:862); here they run
    as runs of 64-token blocks.  Against the oracle at the large block size itself: ragged lengths, skipped and
    duplicated entries, an empty query block; the fused merge against merge(oracle selection)."""
    h = 2
    nqb = -(-n // block)
    q = _randn((1, h, n, 64), n, dtype, 0.5)
    kk = _randn((1, h, n, 64), n + 1, dtype, 0.5)
    v = _randn((1, h, n, 64), n + 2, dtype)
    g = torch.Generator().manual_seed(n + k)
    lo, hi = (-1, nqb + 1) if with_invalid else (0, nqb)
    idx = torch.randint(lo, hi, (1, h, nqb, k), generator=g, dtype=torch.int32)
    if with_invalid:
        idx[0, 0, 0, :] = -1
        if k > 1:
            idx[0, 1, nqb - 1, 1] = idx[0, 1, nqb - 1, 0]
    o = s3r.topk_blocksparse_attention(q.to(DEV), kk.to(DEV), v.to(DEV), idx.to(DEV), block)
    o_ref = oracle.select_attention(q, kk, v, idx, block, out_dtype=torch.float32)
    assert o.dtype == dtype and o.shape == q.shape
    assert max_abs(o, o_ref) <= TOL[dtype]
    if with_invalid:
        assert float(o[0, 0, :min(block, n)].float().abs().max()) == 0.0
    pooled_rows = _randn((1, h, nqb, 64), n + 3, dtype)
    gate = torch.sigmoid(_randn((1, h, n, 2), n + 4, torch.float32)).to(dtype)
    two = s3r.gated_merge(pooled_rows.to(DEV), o, gate.to(DEV), block)
    fused = s3r.select_attn_merge(q.to(DEV), kk.to(DEV), v.to(DEV), idx.to(DEV), pooled_rows.to(DEV), gate.to(DEV), block)
    if dtype == torch.float32:
        assert fused is None                     # the fused epilogue is a 16-bit kernel
    else:                                        # one rounding in the fused epilogue, four in the two operators
        assert merged_within_rounding(fused, pooled_rows.to(DEV), o, gate.to(DEV), block)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_select_block16_handles_scores_far_above_the_reference(dtype):
    """The 16-token kernel fixes a query's softmax reference at the first tile that holds one of its blocks; blocks
    visited later with logits ~140 (base 2) above it overflow the row sums and must send the group through the walk
    with a running maximum.  Also the mild case (probabilities above 1 without overflow: fp16 overflows earlier)."""
    for gain in (12.0, 2.0):
        g = torch.Generator().manual_seed(5)
        n, h = 256, 2
        q = torch.randn((1, h, n, 64), generator=g).to(dtype)
        k = (torch.randn((1, h, n, 64), generator=g) * 0.01).to(dtype)
        k[:, :, 128:192] = (q[:, :, 0:64] * gain).to(dtype)     # key blocks 8..11 line up with the queries of blocks 0..3
        v = torch.randn((1, h, n, 64), generator=g).to(dtype)
        nqb = n // 16
        idx = torch.stack([torch.tensor([(m + 1) % nqb, 8 + (m % 4), (m + 5) % nqb, 9], dtype=torch.int32) for m in range(nqb)])
        idx = idx.view(1, 1, nqb, 4).expand(1, h, nqb, 4).contiguous()
        o = s3r.select_attn(q.to(DEV), k.to(DEV), v.to(DEV), idx.to(DEV), 16)
        ref = oracle.select_attention(q, k, v, idx, 16, out_dtype=torch.float32)
        assert torch.isfinite(o.float()).all()
        assert max_abs(o, ref) <= 2e-2


def test_select_block16_pair_walk_matches_oracle():
    """The cross-check walk of the 16-token kernel (S3R_B16_KERNEL=pairs, read once per process, hence the subprocess)
    against the oracle and against the default union walk: ragged length, skipped and duplicated entries."""
    import subprocess, sys, textwrap
    code = textwrap.dedent("""
        import os, sys, torch
        sys.path.insert(0, ".")
        sys.path.insert(0, "tests")
        import oracle, speed3r_amd as s3r
        n, h, k = 1041, 2, 32
        nqb = -(-n // 16)
        g = torch.Generator().manual_seed(11)
        q, kk, v = ((torch.randn((1, h, n, 64), generator=g) * s).to(torch.bfloat16) for s in (0.5, 0.5, 1.0))
        idx = torch.randint(-1, nqb + 1, (1, h, nqb, k), generator=g, dtype=torch.int32)
        idx[0, 0, 0, :] = -1
        idx[0, 1, 5, 1] = idx[0, 1, 5, 0]
        o = s3r.select_attn(q.cuda(), kk.cuda(), v.cuda(), idx.cuda(), 16)
        ref = oracle.select_attention(q, kk, v, idx, 16, out_dtype=torch.float32)
        err = (o.float().cpu() - ref).abs().max().item()
        assert err <= 2e-2, err
        print("ok", err)
    """)
    env = dict(__import__("os").environ, S3R_B16_KERNEL="pairs")
    res = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=110, env=env)
    assert res.returncode == 0, res.stdout + res.stderr


def test_top64_through_a_banded_score_buffer_equals_the_whole_buffer(monkeypatch):
    """Top-k 64 has no fused index kernel: the scores go through a buffer, a band of query rows at a time once the
    whole matrix would exceed the operator's own buffer limit.  Forced here with a small limit: same bits as with the
    whole buffer, indices equal to the oracle's on the returned scores."""
    from speed3r_amd.sparse_attn import ops
    b, h, l = 1, 3, 700
    q, k, v = (_randn((b, h, l, 64), 40 + i, torch.bfloat16, 0.5).to(DEV) for i in range(3))
    o_ref, idx_ref, scores, lse_ref = ops.compressed_attn_topk(q, k, v, 64, return_scores=True, return_lse=True)
    assert torch.equal(idx_ref.cpu(), torch.from_numpy(oracle.topk_from_scores(scores.cpu().numpy(), 64)))
    monkeypatch.setattr(ops, "SCORE_BUFFER_BYTES", 4 * b * h * l * 256)          # bands of 256 rows: 256, 256, 188
    o, idx, lse = ops.compressed_attn_topk(q, k, v, 64, return_lse=True)
    assert torch.equal(o, o_ref) and torch.equal(idx, idx_ref) and torch.equal(lse, lse_ref)
    qf, kf, vf = (t.float() for t in (q, k, v))                                   # the fp32 instance takes the same route
    o32_ref, idx32_ref = ops.compressed_attn_topk(qf, kf, vf, 16, materialize_scores=True)
    monkeypatch.setattr(ops, "SCORE_BUFFER_BYTES", 4 * b * h * l * 128)
    o32, idx32 = ops.compressed_attn_topk(qf, kf, vf, 16)
    assert torch.equal(o32, o32_ref) and torch.equal(idx32, idx32_ref)


def test_select_with_a_query_row_stride_beyond_the_transfer_offsets():
    """The tile transfers of the MFMA kernels form 32-bit byte offsets from the row strides; a q view whose rows lie
    2^20 elements apart is outside their range and must take the generic kernel: same result as the contiguous q."""
    n, h = 128, 1
    q = _randn((1, h, n, 64), 50, torch.bfloat16, 0.5)
    k = _randn((1, h, n, 64), 51, torch.bfloat16, 0.5).to(DEV)
    v = _randn((1, h, n, 64), 52, torch.bfloat16).to(DEV)
    idx = torch.tensor([[0, 1], [1, 0]], dtype=torch.int32).view(1, 1, 2, 2).to(DEV)
    base = torch.zeros(n * (1 << 20) + 64, dtype=torch.bfloat16, device=DEV)
    q_far = base.as_strided((1, h, n, 64), (0, 0, 1 << 20, 1))
    q_far.copy_(q)
    want = oracle.select_attention(q, k.cpu(), v.cpu(), idx.cpu(), 64, out_dtype=torch.float32)
    assert max_abs(s3r.select_attn(q_far, k, v, idx, 64), want) <= 2e-2
    assert max_abs(s3r.select_attn(q.to(DEV), k, v, idx, 64), want) <= 2e-2


def test_select_block16_rows_beyond_4_gib_from_the_tensor_start():
    """16-token blocks on K and V views whose last rows lie more than 4 GiB behind the first (row stride just below
    2^20 elements, 2112 rows): every transfer instruction addresses its rows from a descriptor based at the block, so
    the byte offsets stay small whatever the tensor's extent.  (The layer passes V as the in-place view of the packed
    projection, 6 KB per row: the same holds there from 700 000 tokens on.)"""
    n, h, kk, stride = 2112, 1, 8, (1 << 20) - 64
    q = _randn((1, h, n, 64), 60, torch.bfloat16, 0.5)
    k = _randn((1, h, n, 64), 61, torch.bfloat16, 0.5)
    v = _randn((1, h, n, 64), 62, torch.bfloat16)
    nqb = n // 16
    idx = torch.randint(-1, nqb, (1, h, nqb, kk), generator=torch.Generator().manual_seed(63), dtype=torch.int32)
    idx[..., 0] = nqb - 1 - torch.arange(nqb, dtype=torch.int32) % 8          # every query block reads from the far end
    far = []
    for t in (k, v):
        base = torch.empty(n * stride + 64, dtype=torch.bfloat16, device=DEV)
        view = base.as_strided((1, h, n, 64), (0, 0, stride, 1))
        view.copy_(t)
        far.append(view)
    assert (n - 1) * stride * 2 > (1 << 32)
    got = s3r.select_attn(q.to(DEV), far[0], far[1], idx.to(DEV), 16)
    want = oracle.select_attention(q, k, v, idx, 16, out_dtype=torch.float32)
    assert max_abs(got, want) <= 2e-2
    del far
    torch.cuda.empty_cache()
