"""Parity of the attention backward kernels against the CPU oracle, through the C-ABI (needs an MI355X).

Bar: bf16/fp16 gradients within 2e-2 * max(1, max|reference|) of the oracle's fp32/fp64 gradients on the same
(already rounded) inputs.  The device forward supplies o and lse, as in training.
"""
import pytest
import torch

import oracle
import speed3r_amd as s3r
from speed3r_amd.sparse_attn import ops
from helpers import max_abs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _randn(shape, seed, dtype, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def _close(got, want, what):
    tol = 2e-2 * max(1.0, float(want.abs().max()))
    err = max_abs(got, want)
    assert err <= tol, f"{what}: max abs error {err:.4g} > {tol:.4g}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n", [128, 200, 64, 333])
def test_delta_is_the_row_dot_product(dtype, n):
    o, g = _randn((2, 3, n, 64), 1, dtype), _randn((2, 3, n, 64), 2, dtype)
    got = ops.attn_bwd_delta(o.to(DEV), g.to(DEV))
    want = (o.float() * g.float()).sum(-1)
    assert max_abs(got, want) <= 1e-4


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("lq,lk", [(128, 128), (200, 200), (70, 70), (64, 64), (521, 521)])
def test_dense_backward_matches_oracle(dtype, lq, lk):
    q, k, v = (_randn((1, 2, l, 64), 10 + i, dtype, 0.5) for i, l in enumerate((lq, lk, lk)))
    g = _randn((1, 2, lq, 64), 20, dtype)
    qd, kd, vd, gd = (t.to(DEV) for t in (q, k, v, g))
    o, _, lse = s3r.compressed_attn_topk(qd, kd, vd, None, return_lse=True)
    dq, dk, dv = ops.attn_bwd(qd, kd, vd, o, gd, lse)
    wq, wk, wv = oracle.compressed_attention_grads_autograd(q, k, v, g)
    _close(dq, wq, "dq"); _close(dk, wk, "dk"); _close(dv, wv, "dv")


def _rand_idx(b, h, nqb, kk, nkb, seed, lo=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, nkb, (b, h, nqb, kk), generator=g, dtype=torch.int32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,kk", [(512, 4), (1000, 4), (1041, 8), (256, 1), (4100, 16)])
def test_selection_backward_matches_oracle(dtype, n, kk):
    b, h = 1, 2
    nqb = -(-n // 64)
    q, k, v, g = (_randn((b, h, n, 64), 30 + i, dtype, 0.5 if i < 3 else 1.0) for i in range(4))
    idx = _rand_idx(b, h, nqb, kk, nqb, 40 + n)
    qd, kd, vd, gd, idxd = (t.to(DEV) for t in (q, k, v, g, idx))
    o, lse = s3r.select_attn(qd, kd, vd, idxd, 64, return_lse=True)
    dq, dk, dv = ops.attn_bwd(qd, kd, vd, o, gd, lse, idxd)
    wq, wk, wv = oracle.select_attention_grads_autograd(q, k, v, idx, 64, g)
    _close(dq, wq, "dq"); _close(dk, wk, "dk"); _close(dv, wv, "dv")


def test_selection_backward_with_skips_duplicates_and_unattended_keys():
    b, h, n, kk = 1, 2, 640, 4
    nqb = n // 64
    q, k, v, g = (_randn((b, h, n, 64), 50 + i, torch.bfloat16, 0.5 if i < 3 else 1.0) for i in range(4))
    idx = _rand_idx(b, h, nqb, kk, nqb - 2, 55, lo=-1)       # -1 entries; key blocks 8, 9 are never attended
    idx[0, 0, 2] = torch.tensor([3, 3, 3, 1])                   # duplicates
    idx[0, 1, 4] = -1                                           # a query block that attends nothing
    idx[0, 1, 5, 0] = nqb + 3                                   # beyond the sequence: skipped
    qd, kd, vd, gd, idxd = (t.to(DEV) for t in (q, k, v, g, idx))
    o, lse = s3r.select_attn(qd, kd, vd, idxd, 64, return_lse=True)
    dq, dk, dv = ops.attn_bwd(qd, kd, vd, o, gd, lse, idxd)
    mult = oracle.block_multiplicity(idx, n, 64)
    wq, wk, wv, _, _ = oracle.attention_grads_formula(q, k, v, g, mult)
    _close(dq, wq, "dq"); _close(dk, wk, "dk"); _close(dv, wv, "dv")
    assert float(dq[0, 1, 256:320].abs().max()) == 0.0                    # the empty query block
    assert float(dk[0, :, 512:].abs().max()) == 0.0 and float(dv[0, :, 512:].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,kk", [(256, 4), (1000, 8), (1041, 32), (64, 2), (40, 1), (2100, 16)])
def test_selection_backward_with_16_token_blocks_matches_oracle(dtype, n, kk):
    """Block 16, the reference layer's own setting (sparse_attention.py:73,98): sequence lengths that are no multiple
    of 16 or of 64, so ragged blocks and partly filled 64-row tiles are covered."""
    b, h = 1, 2
    nqb = -(-n // 16)
    q, k, v, g = (_randn((b, h, n, 64), 130 + i, dtype, 0.5 if i < 3 else 1.0) for i in range(4))
    idx = _rand_idx(b, h, nqb, kk, nqb, 140 + n)
    qd, kd, vd, gd, idxd = (t.to(DEV) for t in (q, k, v, g, idx))
    o, lse = s3r.select_attn(qd, kd, vd, idxd, 16, return_lse=True)
    dq, dk, dv = ops.attn_bwd(qd, kd, vd, o, gd, lse, idxd, 16)
    wq, wk, wv = oracle.select_attention_grads_autograd(q, k, v, idx, 16, g)
    _close(dq, wq, "dq"); _close(dk, wk, "dk"); _close(dv, wv, "dv")


def test_selection_backward_with_16_token_blocks_skips_duplicates_and_popular_keys():
    b, h, n, kk = 1, 2, 400, 4
    nqb = n // 16
    q, k, v, g = (_randn((b, h, n, 64), 150 + i, torch.bfloat16, 0.5 if i < 3 else 1.0) for i in range(4))
    idx = _rand_idx(b, h, nqb, kk, nqb - 3, 155, lo=-1)       # -1 entries; the last three key blocks are never attended
    idx[0, 0, 2] = torch.tensor([3, 3, 3, 1])                   # duplicates
    idx[0, 1, 4] = -1                                           # a query block that attends nothing
    idx[0, 1, 5, 0] = nqb + 3                                   # beyond the sequence: skipped
    idx[0, 0, :, 1] = 7                                         # one key block on every list: lists of unequal length
    qd, kd, vd, gd, idxd = (t.to(DEV) for t in (q, k, v, g, idx))
    o, lse = s3r.select_attn(qd, kd, vd, idxd, 16, return_lse=True)
    dq, dk, dv = ops.attn_bwd(qd, kd, vd, o, gd, lse, idxd, 16)
    mult = oracle.block_multiplicity(idx, n, 16)
    wq, wk, wv, _, _ = oracle.attention_grads_formula(q, k, v, g, mult)
    _close(dq, wq, "dq"); _close(dk, wk, "dk"); _close(dv, wv, "dv")
    assert float(dq[0, 1, 64:80].abs().max()) == 0.0                      # the empty query block
    assert float(dk[0, :, 16 * (nqb - 3):].abs().max()) == 0.0 and float(dv[0, :, 16 * (nqb - 3):].abs().max()) == 0.0


@pytest.mark.parametrize("n,kk", [(1040, 2), (2000, 4), (650, 1)])
def test_selection_backward_with_16_token_blocks_and_very_long_lists(n, kk):
    """Key blocks that nearly every query block lists: the union of their workgroup's four lists is built in several
    chunks (a list offers 96 entries per chunk), next to ordinary tiles and a ragged last block."""
    b, h = 1, 2
    nqb = -(-n // 16)
    q, k, v, g = (_randn((b, h, n, 64), 170 + i, torch.bfloat16, 0.5 if i < 3 else 1.0) for i in range(4))
    idx = _rand_idx(b, h, nqb, kk, nqb, 175 + n)
    idx[0, 0, :, 0] = 9                        # on every list of head 0
    idx[0, 1, ::2, 0] = nqb - 1                # the ragged last block on every second list of head 1
    idx[0, 1, 1::2, 0] = 3
    qd, kd, vd, gd, idxd = (t.to(DEV) for t in (q, k, v, g, idx))
    o, lse = s3r.select_attn(qd, kd, vd, idxd, 16, return_lse=True)
    dq, dk, dv = ops.attn_bwd(qd, kd, vd, o, gd, lse, idxd, 16)
    mult = oracle.block_multiplicity(idx, n, 16)
    wq, wk, wv, _, _ = oracle.attention_grads_formula(q, k, v, g, mult)
    _close(dq, wq, "dq"); _close(dk, wk, "dk"); _close(dv, wv, "dv")


def test_selection_backward_with_16_token_blocks_and_long_lists_side_by_side():
    """Four neighbouring key blocks of one workgroup with long lists of different lengths (all, every second, every
    third query block, a run in the middle), one of them named twice by some query blocks: every chunk of the union
    takes entries from several lists, and the chunk borders fall differently in each."""
    b, h, n, kk = 1, 2, 4000, 6
    nqb = n // 16
    q, k, v, g = (_randn((b, h, n, 64), 190 + i, torch.bfloat16, 0.5 if i < 3 else 1.0) for i in range(4))
    idx = _rand_idx(b, h, nqb, kk, nqb, 195)
    idx[0, 0, :, 0] = 8                        # key blocks 8..11 are one workgroup's
    idx[0, 0, ::2, 1] = 9
    idx[0, 0, ::3, 2] = 10
    idx[0, 0, 60:200, 3] = 11
    idx[0, 0, 100:130, 4] = 8                  # ... and 8 twice on these lists
    idx[0, 1, :, 0] = 41                       # head 1: two long lists in different workgroups' neighbourhoods
    idx[0, 1, 5:, 1] = 43
    qd, kd, vd, gd, idxd = (t.to(DEV) for t in (q, k, v, g, idx))
    o, lse = s3r.select_attn(qd, kd, vd, idxd, 16, return_lse=True)
    dq, dk, dv = ops.attn_bwd(qd, kd, vd, o, gd, lse, idxd, 16)
    mult = oracle.block_multiplicity(idx, n, 16)
    wq, wk, wv, _, _ = oracle.attention_grads_formula(q, k, v, g, mult)
    _close(dq, wq, "dq"); _close(dk, wk, "dk"); _close(dv, wv, "dv")


@pytest.mark.parametrize("b,h,nqb,kk,nkb,hot", [(2, 3, 37, 4, 37, 0), (1, 2, 300, 8, 300, 1), (1, 1, 2600, 4, 650, 2),
                                                (1, 2, 9000, 2, 40, 3), (1, 1, 1, 1, 1, 0), (1, 2, 70, 64, 70, 0)])
def test_key_block_lists_match_plain_loops(b, h, nqb, kk, nkb, hot):
    """The device lists against the oracle's plain loops: entries outside [0, nkb), duplicates, lists of up to 512
    entries (sorted by one wavefront), of more (by a workgroup in LDS; hot == 2) and of more than 8192 (in global
    memory; hot == 3), and the same bits on a second run (the atomic order of the fill must not show)."""
    gen = torch.Generator().manual_seed(22 + nqb)
    idx = torch.randint(-2, nkb + 2, (b, h, nqb, kk), generator=gen, dtype=torch.int32)
    if hot >= 1:
        idx[0, 0, :, 0] = 5                      # a key block on every index row
    if hot >= 2:
        idx[0, 0, ::3, 1] = 5                    # ... twice on every third
    if hot >= 3:
        idx[0, 1] = 7                            # nqb * K = 18 000 entries in one list
    idx[-1, -1, nqb // 2] = 1
    lists, off = ops.key_block_lists(idx.to(DEV), nkb)
    lists2, off2 = ops.key_block_lists(idx.to(DEV), nkb)
    want = oracle.key_block_lists(idx, nkb)
    assert lists.dtype == torch.int32 and off.dtype == torch.int32 and off.shape == (b, h, nkb + 1)
    assert torch.equal(off, off2)
    off, lists, lists2 = off.cpu(), lists.cpu(), lists2.cpu()
    for bh in range(b * h):
        o = off.view(b * h, nkb + 1)[bh].tolist()
        flat = lists.view(b * h, -1)[bh].tolist()
        assert o[0] == 0 and flat[:o[-1]] == lists2.view(b * h, -1)[bh].tolist()[:o[-1]]
        for j in range(nkb):
            assert flat[o[j]:o[j + 1]] == want[bh][j], (bh, j)


@pytest.mark.parametrize("name,block", [("b16", 16), ("b64", 64)])
def test_selection_forward_and_backward_match_the_brute_force_fixture(golden_grads, name, block):
    from helpers import from_bf16_bits

    q, k, v, g = (from_bf16_bits(golden_grads[n]).to(DEV) for n in ("q", "k", "v", "dout"))
    idx = torch.from_numpy(golden_grads[f"{name}_idx"]).to(DEV)
    o, lse = s3r.select_attn(q, k, v, idx, block, return_lse=True)
    assert max_abs(o, torch.from_numpy(golden_grads[f"{name}_out"])) <= 2e-2
    dq, dk, dv = ops.attn_bwd(q, k, v, o, g, lse, idx, block)
    for got, t in ((dq, "dq"), (dk, "dk"), (dv, "dv")):
        _close(got, torch.from_numpy(golden_grads[f"{name}_{t}"]), t)


def test_operators_are_differentiable_like_the_reference_ones():
    b, h, n = 1, 2, 512
    q, k, v = (_randn((b, h, n, 64), 60 + i, torch.bfloat16, 0.5).to(DEV).requires_grad_(True) for i in range(3))
    g = _randn((b, h, n, 64), 63, torch.bfloat16).to(DEV)
    idx = _rand_idx(b, h, n // 64, 4, n // 64, 64).to(DEV)
    o = s3r.topk_blocksparse_attention(q, k, v, idx, 64)
    o.backward(g)
    with torch.no_grad():
        o2, lse = s3r.select_attn(q, k, v, idx, 64, return_lse=True)
        dq, dk, dv = ops.attn_bwd(q, k, v, o2, g, lse, idx)
    assert torch.equal(o, o2) and torch.equal(q.grad, dq) and torch.equal(k.grad, dk) and torch.equal(v.grad, dv)
    # compressed branch: gradients flow through the attention output, the indices carry none
    qc, kc, vc = (_randn((b, h, 100, 64), 70 + i, torch.bfloat16, 0.5).to(DEV).requires_grad_(True) for i in range(3))
    gc = _randn((b, h, 100, 64), 73, torch.bfloat16)
    oc, ic = s3r.flash_attn_topk_func(qc, kc, vc, 4)
    assert not ic.requires_grad and ic.dtype == torch.int32
    oc.backward(gc.to(DEV))
    wq, wk, wv = oracle.compressed_attention_grads_autograd(qc.detach().cpu(), kc.detach().cpu(), vc.detach().cpu(), gc)
    _close(qc.grad, wq, "dq"); _close(kc.grad, wk, "dk"); _close(vc.grad, wv, "dv")
    # only q wants a gradient: the dk/dv kernel is skipped
    q2 = q.detach().clone().requires_grad_(True)
    s3r.topk_blocksparse_attention(q2, k.detach(), v.detach(), idx, 64).backward(g)
    assert torch.equal(q2.grad, dq)


def test_backward_is_linear_in_the_output_gradient_and_sums_over_value_columns():
    b, h, n, kk = 1, 4, 2048, 8
    q, k, v, g = (_randn((b, h, n, 64), 80 + i, torch.bfloat16, 0.5 if i < 3 else 1.0).to(DEV) for i in range(4))
    idx = _rand_idx(b, h, n // 64, kk, n // 64, 85).to(DEV)
    o, lse = s3r.select_attn(q, k, v, idx, 64, return_lse=True)
    dq, dk, dv = ops.attn_bwd(q, k, v, o, g, lse, idx)
    dq2, dk2, dv2 = ops.attn_bwd(q, k, v, o, 2 * g, lse, idx)
    for a, c2 in ((dq, dq2), (dk, dk2), (dv, dv2)):
        assert max_abs(2 * a.float(), c2) <= 2e-2 * max(1.0, float(c2.float().abs().max()))
    # P sums to one over the attended keys: the column sums of dV equal those of dO (every query block attends something)
    assert max_abs(dv.float().sum(2), g.float().sum(2)) <= 0.05 * float(g.float().sum(2).abs().max())


def test_backward_at_full_size_on_sampled_blocks():
    # 266 496 tokens, 16 heads, top-k 16 (the headline shape): gradients of sampled query blocks (dq) and key blocks
    # (dk, dv) against an fp32 restatement of the formulas on the device
    from speed3r_amd import workloads

    cfg, q, k, v, _ = workloads.make_config("cfg3")
    n, nb, kk = cfg.tokens, cfg.tokens // 64, cfg.topk
    q, k, v = (t.to(DEV) for t in (q, k, v))
    qc, kc, vc = (s3r.pool_mean(t, 64) for t in (q, k, v))
    _, idx = s3r.compressed_attn_topk(qc, kc, vc, kk)
    o, lse = s3r.select_attn(q, k, v, idx, 64, return_lse=True)
    g = torch.randn(o.shape, generator=torch.Generator().manual_seed(90)).to(torch.bfloat16).to(DEV)
    dq, dk, dv = ops.attn_bwd(q, k, v, o, g, lse, idx)
    assert torch.isfinite(dq.float()).all() and torch.isfinite(dk.float()).all() and torch.isfinite(dv.float()).all()
    delta = (o.float() * g.float()).sum(-1)                                           # [1, 16, n]
    lists, off = ops.key_block_lists(idx, nb)
    gen = torch.Generator().manual_seed(91)
    ar = torch.arange(64, device=DEV)
    for m in torch.randint(0, nb, (6,), generator=gen).tolist():                      # query blocks
        rows = slice(64 * m, 64 * m + 64)
        tok = (idx[0, :, m].long()[:, :, None] * 64 + ar).reshape(16, kk * 64)        # [16 heads, K*64] key tokens
        kg = k[0].gather(1, tok[:, :, None].expand(16, kk * 64, 64)).float()
        vg = v[0].gather(1, tok[:, :, None].expand(16, kk * 64, 64)).float()
        p = torch.exp(q[0, :, rows].float() @ kg.transpose(1, 2) / 8.0 - lse[0, :, rows, None])
        ds = p * (g[0, :, rows].float() @ vg.transpose(1, 2) - delta[0, :, rows, None]) / 8.0
        want = ds @ kg
        assert max_abs(dq[0, :, rows], want) <= 2e-2 * max(1.0, float(want.abs().max()))
    for j in torch.randint(0, nb, (6,), generator=gen).tolist():                      # key blocks
        keys = slice(64 * j, 64 * j + 64)
        for h in (0, 7, 15):
            lo, hi = int(off[0, h, j]), int(off[0, h, j + 1])
            want_dk = torch.zeros((64, 64), device=DEV)
            want_dv = torch.zeros((64, 64), device=DEV)
            if hi > lo:
                qtok = (lists[0, h, lo:hi].long()[:, None] * 64 + ar).reshape(-1)     # query tokens attending block j
                qf, gf = q[0, h, qtok].float(), g[0, h, qtok].float()
                p = torch.exp(qf @ k[0, h, keys].float().T / 8.0 - lse[0, h, qtok, None])
                ds = p * (gf @ v[0, h, keys].float().T - delta[0, h, qtok, None]) / 8.0
                want_dk, want_dv = ds.T @ qf, p.T @ gf
            assert max_abs(dk[0, h, keys], want_dk) <= 2e-2 * max(1.0, float(want_dk.abs().max()))
            assert max_abs(dv[0, h, keys], want_dv) <= 2e-2 * max(1.0, float(want_dv.abs().max()))


@pytest.mark.parametrize("n,block,kk", [(1041, 128, 3), (1500, 256, 2)])
def test_selection_backward_with_blocks_of_128_and_256_tokens(n, block, kk):
    """The differentiable operator at the reference's larger block sizes (run as runs of 64-token blocks) against
    autograd through the oracle at the large block size itself."""
    b, h, dtype = 1, 2, torch.bfloat16
    nqb = -(-n // block)
    q, k, v, g = (_randn((b, h, n, 64), 60 + i, dtype, 0.5 if i < 3 else 1.0) for i in range(4))
    idx = _rand_idx(b, h, nqb, kk, nqb, 70 + n)
    qd, kd, vd = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    o = s3r.topk_blocksparse_attention(qd, kd, vd, idx.to(DEV), block)
    o.backward(g.to(DEV))
    wq, wk, wv = oracle.select_attention_grads_autograd(q, k, v, idx, block, g)
    _close(qd.grad, wq, "dq"); _close(kd.grad, wk, "dk"); _close(vd.grad, wv, "dv")


def test_caller_built_lists_that_are_not_ascending_are_refused_on_request():
    """ops.attn_bwd(check_lists=True): lists from key_block_lists pass; the same lists with one group reversed raise
    (without the check the 16-token dK/dV kernel would skip entries and return incomplete gradients silently)."""
    import pytest as _pytest
    from speed3r_amd.sparse_attn import ops
    g = torch.Generator().manual_seed(3)
    n, h, kk, block = 256, 1, 4, 16
    q, k, v = ((torch.randn((1, h, n, 64), generator=g) * 0.5).to(torch.bfloat16).to("cuda:0") for _ in range(3))
    nqb = n // block
    idx = torch.stack([torch.randperm(nqb, generator=g)[:kk] for _ in range(nqb)]).to(torch.int32).view(1, h, nqb, kk).to("cuda:0")
    o, lse = ops.select_attn(q, k, v, idx, block, return_lse=True)
    dout = torch.randn(o.shape, generator=g).to(torch.bfloat16).to("cuda:0")
    lists, offs = ops.key_block_lists(idx, nqb)
    want = ops.attn_bwd(q, k, v, o, dout, lse, idx, block, key_lists=(lists, offs), check_lists=True)
    ref = ops.attn_bwd(q, k, v, o, dout, lse, idx, block)
    assert all(torch.equal(a, b) for a, b in zip(want, ref))
    lens = (offs[0, 0, 1:] - offs[0, 0, :-1]).cpu()
    j = int(torch.nonzero(lens >= 2)[0])
    lo, hi = int(offs[0, 0, j]), int(offs[0, 0, j + 1])
    bad = lists.clone()
    bad[0, 0, lo:hi] = lists[0, 0, lo:hi].flip(0)
    assert not ops.key_lists_ascending(bad, offs)
    with _pytest.raises(ValueError, match="ascending"):
        ops.attn_bwd(q, k, v, o, dout, lse, idx, block, key_lists=(bad, offs), check_lists=True)
