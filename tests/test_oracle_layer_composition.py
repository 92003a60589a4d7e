"""Pins of ``oracle.sparse_layer`` -- the composition of the layer around the two operators
(reference pi3/models/layers/sparse_attention.py:90-141).

Nothing in the reference holds an output of the layer, so the composition is pinned by what the mathematics fixes:
when every key block is selected the selection branch IS dense attention, so the layer must equal

    proj( g0 * broadcast(compressed row of the token's block) + g1 * dense_attention )

with every factor built HERE from explicit per-head weight slices (the meaning of the reference's einops patterns
``'b n (qkv h d)'`` at :97 and ``'b n (h g)'`` at :94 spelled out as row ranges of the weight matrices), library
routines (``F.layer_norm``, ``F.scaled_dot_product_attention``), the textbook rotation written with complex numbers
and plain block means.  With fewer blocks selected the selection branch is a block-masked dense softmax whose mask
comes from ``torch.topk`` of the pooled scores.  Each expected value is built by a function that can also be asked
for a plausible MISTAKE (a swapped split order, a swapped gate pairing, norm before pooling, rounded mean block
positions ...); every test asserts both that the oracle equals the correct construction and that each mistaken one
is far outside the tolerance, so a test that would not notice the mistake cannot pass.
"""
import math

import pytest
import torch
import torch.nn.functional as F

import oracle

TOL = 3e-5            # fp32 composition of ~5 matmuls on O(1) values
FAR = 1e-2            # a wrong composition is at least this far away


def _params(dim, heads, seed, qk_norm=True, gate_scale=1.0):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g)
    d = dim // heads
    p = dict(w_qkv=r(3 * dim, dim) / math.sqrt(dim), b_qkv=0.1 * r(3 * dim),
             w_gate=gate_scale * r(2 * heads, dim) / math.sqrt(dim), b_gate=gate_scale * r(2 * heads),
             w_proj=r(dim, dim) / math.sqrt(dim), b_proj=0.1 * r(dim))
    if qk_norm:
        p.update(qn_w=1 + 0.3 * r(d), qn_b=0.2 * r(d), kn_w=1 + 0.3 * r(d), kn_b=0.2 * r(d))
    return p


def _grid_positions(b, n, width):
    """Row-major (y, x) patch positions of a ``width``-wide grid, as PositionGetter gives them (pos_embed.py:162-174)."""
    t = torch.arange(n)
    return torch.stack((t // width, t % width), dim=-1)[None].expand(b, -1, -1).contiguous()


def _rotate(t, coord, base):
    """Textbook rotary embedding of one half (the y or x part) by integer coordinates, with complex numbers:
    element j pairs with element j + len/2, frequency base**(-2j/len)."""
    half = t.shape[-1] // 2
    freq = base ** (-torch.arange(half, dtype=torch.float64) * 2 / t.shape[-1])
    z = torch.complex(t[..., :half].double(), t[..., half:].double())
    ang = coord.double()[:, None, :, None] * freq
    z = z * torch.polar(torch.ones_like(ang), ang)
    return torch.cat((z.real, z.imag), dim=-1).float()


def _rope(t, pos, base=100.0):
    d = t.shape[-1]
    return torch.cat((_rotate(t[..., :d // 2], pos[..., 0], base), _rotate(t[..., d // 2:], pos[..., 1], base)), dim=-1)


def _expected(x, p, heads, block, xpos, mistake=None, keep=None):
    """The layer from first principles.  ``keep``: number of key blocks each query block attends to in the
    selection branch (None: all of them -> dense attention)."""
    b, n, c = x.shape
    d = c // heads
    nc = n // block
    cols = []
    for h in range(heads):
        def rows(which):                       # rows of the packed projection that give head h of q (0), k (1), v (2)
            if mistake == "split_h_qkv_d":     # '(h qkv d)' instead of '(qkv h d)'
                lo = h * 3 * d + which * d
            elif mistake == "split_kqv":       # k and q exchanged
                lo = {0: 1, 1: 0, 2: 2}[which] * c + h * d
            else:
                lo = which * c + h * d
            return slice(lo, lo + d)
        q, k, v = (x @ p["w_qkv"][rows(i)].T + p["b_qkv"][rows(i)] for i in range(3))          # [B,N,D] each
        g_rows = (h, heads + h) if mistake == "gate_g_h" else (2 * h, 2 * h + 1)               # '(g h)' vs '(h g)'
        g0, g1 = (torch.sigmoid(x @ p["w_gate"][r] + p["b_gate"][r]) for r in g_rows)          # [B,N] each
        if mistake == "gate_swapped":
            g0, g1 = g1, g0

        def norm(t, which):
            if "qn_w" not in p:
                return t
            w, bias = (p["qn_w"], p["qn_b"]) if which == 0 else (p["kn_w"], p["kn_b"])
            if mistake == "norm_params_swapped":
                w, bias = (p["kn_w"], p["kn_b"]) if which == 0 else (p["qn_w"], p["qn_b"])
            return F.layer_norm(t, (d,), w, bias)

        def pooled(t):
            return t.view(b, nc, block, d).mean(dim=2)

        # compressed branch: pool the RAW projection, then norm, then rotate at the truncated mean block position
        if mistake == "norm_before_pool":
            qc, kc = pooled(norm(q, 0)), pooled(norm(k, 1))
        else:
            qc, kc = norm(pooled(q), 0), norm(pooled(k), 1)
        vc = pooled(v)
        if xpos is not None:
            mean_pos = xpos.view(b, nc, block, 2).float().mean(dim=2)
            pc = mean_pos.round().long() if mistake == "block_pos_rounded" else mean_pos.long()
            if mistake == "block_pos_first":
                pc = xpos.view(b, nc, block, 2)[:, :, 0]
            qc, kc = _rope(qc[:, None], pc)[:, 0], _rope(kc[:, None], pc)[:, 0]
        s_c = qc @ kc.transpose(1, 2)                                                            # raw pooled scores
        o_c = torch.softmax(s_c / math.sqrt(d), dim=-1) @ vc                                     # [B,Nc,D]

        # full-token branch
        qf, kf = norm(q, 0), norm(k, 1)
        if xpos is not None and mistake != "no_token_rope":
            px = xpos.flip(-1) if mistake == "xy_swapped" else xpos
            qf, kf = _rope(qf[:, None], px)[:, 0], _rope(kf[:, None], px)[:, 0]
        if keep is None:
            o_s = F.scaled_dot_product_attention(qf[:, None], kf[:, None], v[:, None])[:, 0]
        else:
            top = torch.topk(s_c, keep, dim=-1).indices                                          # [B,Nc,keep]
            allowed = torch.zeros((b, nc, nc), dtype=torch.bool).scatter_(2, top, True)
            mask = allowed.repeat_interleave(block, dim=1).repeat_interleave(block, dim=2)       # [B,N,N]
            s = (qf @ kf.transpose(1, 2)) / math.sqrt(d)
            o_s = torch.softmax(s.masked_fill(~mask, float("-inf")), dim=-1) @ v
        o_c_tok = o_c.repeat_interleave(block, dim=1)                                            # the token's block row
        cols.append(g0[..., None] * o_c_tok + g1[..., None] * o_s)
    merged = torch.cat(cols, dim=-1)                                                             # 'b n (h d)'
    if mistake == "merge_d_h":
        merged = torch.stack(cols, dim=-1).reshape(b, n, c)
    return merged @ p["w_proj"].T + p["b_proj"]


def _oracle(x, p, heads, block, topk, xpos):
    return oracle.sparse_layer(x, p["w_qkv"], p["b_qkv"], p["w_gate"], p["b_gate"], p["w_proj"], p["b_proj"],
                               heads, block, topk, xpos=xpos, qn_w=p.get("qn_w"), qn_b=p.get("qn_b"),
                               kn_w=p.get("kn_w"), kn_b=p.get("kn_b"))


MISTAKES = ["split_h_qkv_d", "split_kqv", "gate_g_h", "gate_swapped", "norm_params_swapped", "norm_before_pool",
            "block_pos_first", "no_token_rope", "xy_swapped", "merge_d_h"]


def _case(seed, b=2, heads=2, d=16, block=8, nc=8, width=6, qk_norm=True):
    dim = heads * d
    n = nc * block
    g = torch.Generator().manual_seed(100 + seed)
    x = torch.randn(b, n, dim, generator=g)
    return x, _params(dim, heads, seed, qk_norm), heads, block, _grid_positions(b, n, width)


@pytest.mark.parametrize("seed", [0, 1])
def test_with_every_block_selected_the_layer_is_gated_compressed_plus_dense_attention(seed):
    x, p, heads, block, xpos = _case(seed)
    nc = x.shape[1] // block
    got = _oracle(x, p, heads, block, nc, xpos)
    assert sorted(got["idx"][0, 0, 0].tolist()) == list(range(nc))            # every block once
    want = _expected(x, p, heads, block, xpos)
    assert (got["out"] - want).abs().max().item() <= TOL
    for m in MISTAKES:
        wrong = _expected(x, p, heads, block, xpos, mistake=m)
        assert (got["out"] - wrong).abs().max().item() >= FAR, m


def test_truncated_not_rounded_block_positions():
    # width 5, block 8: block means have fractional parts above one half in x, where int() and round() differ
    x, p, heads, block, xpos = _case(2, width=5)
    got = _oracle(x, p, heads, block, x.shape[1] // block, xpos)
    assert (got["out"] - _expected(x, p, heads, block, xpos)).abs().max().item() <= TOL
    frac = xpos.view(2, -1, block, 2).float().mean(2) % 1
    assert (frac > 0.5).any()
    assert (got["out"] - _expected(x, p, heads, block, xpos, mistake="block_pos_rounded")).abs().max().item() >= 1e-3


def test_gate_extremes_isolate_each_branch():
    """Gate driven to (0, 1): the layer is the reference's eager dense layer (sparse_attention.py:39-58);
    gate driven to (1, 0): the output is proj of each block's compressed row broadcast over its tokens."""
    x, p, heads, block, xpos = _case(3)
    nc = x.shape[1] // block
    p["w_gate"] = torch.zeros_like(p["w_gate"])
    for pair, branch in (((-60.0, 60.0), "dense"), ((60.0, -60.0), "compressed")):
        p["b_gate"] = torch.tensor(pair).repeat(heads)                          # the reference's own (h g) bias layout, :79
        got = _oracle(x, p, heads, block, nc, xpos)
        want = _expected(x, p, heads, block, xpos)
        assert (got["out"] - want).abs().max().item() <= TOL
        merged = torch.linalg.solve(p["w_proj"], (got["out"] - p["b_proj"]).transpose(1, 2)).transpose(1, 2)
        per_block = merged.view(2, nc, block, -1)
        spread = (per_block - per_block[:, :, :1]).abs().max().item()
        if branch == "compressed":
            assert spread <= 1e-3                                               # one row per block, broadcast
        else:
            assert spread >= 0.05                                               # token-wise attention output
            b, n, c = x.shape
            qkv = F.linear(x, p["w_qkv"], p["b_qkv"]).reshape(b, n, 3, heads, c // heads).permute(2, 0, 3, 1, 4)
            q = F.layer_norm(qkv[0], (c // heads,), p["qn_w"], p["qn_b"])
            k = F.layer_norm(qkv[1], (c // heads,), p["kn_w"], p["kn_b"])
            q, k = oracle.rope2d(q, xpos), oracle.rope2d(k, xpos)
            dense = F.scaled_dot_product_attention(q, k, qkv[2]).transpose(1, 2).reshape(b, n, c)
            assert (got["out"] - F.linear(dense, p["w_proj"], p["b_proj"])).abs().max().item() <= TOL


@pytest.mark.parametrize("keep", [1, 2, 4])
def test_with_fewer_blocks_the_selection_branch_is_the_block_masked_softmax_of_the_pooled_top_scores(keep):
    x, p, heads, block, xpos = _case(4 + keep, nc=16)
    got = _oracle(x, p, heads, block, keep, xpos)
    want = _expected(x, p, heads, block, xpos, keep=keep)
    assert (got["out"] - want).abs().max().item() <= TOL
    for m in ("split_kqv", "norm_before_pool", "block_pos_first", "gate_g_h"):
        wrong = _expected(x, p, heads, block, xpos, mistake=m, keep=keep)
        assert (got["out"] - wrong).abs().max().item() >= FAR, m


def test_without_qk_norm_and_without_positions():
    x, p, heads, block, _ = _case(9, qk_norm=False)
    got = _oracle(x, p, heads, block, 2, None)
    assert (got["out"] - _expected(x, p, heads, block, None, keep=2)).abs().max().item() <= TOL


def test_reference_initial_gate_weights_both_branches_by_sigmoid_of_minus_and_plus_one():
    """At the reference's initial gate (weight 0, bias (-1, 1) per head, :76-80) the merge is
    0.26894 * compressed + 0.73106 * selection for every token."""
    x, p, heads, block, xpos = _case(10)
    nc = x.shape[1] // block
    p["w_gate"] = torch.zeros_like(p["w_gate"])
    p["b_gate"] = torch.tensor([-1.0, 1.0]).repeat(heads)
    got = _oracle(x, p, heads, block, nc, xpos)
    merged = oracle.gated_merge(got["o_cmp"], got["o_sel"], torch.tensor([0.2689414, 0.7310586]).expand(2, heads, x.shape[1], 2), block)
    assert (got["out"] - F.linear(merged, p["w_proj"], p["b_proj"])).abs().max().item() <= TOL
    assert (got["out"] - _expected(x, p, heads, block, xpos)).abs().max().item() <= TOL
