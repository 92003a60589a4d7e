"""The layer module (speed3r_amd.layers.SparseFlashAttentionRope) on the GPU against the CPU layer oracle."""
import pytest
import torch

import oracle
from helpers import max_abs
from speed3r_amd.layers import RoPE2D, SparseFlashAttentionRope

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _make(dim, heads, block_size, topk, dtype, seed, qk_norm=True):
    torch.manual_seed(seed)
    m = SparseFlashAttentionRope(dim=dim, num_heads=heads, qkv_bias=True, qk_norm=qk_norm, rope=RoPE2D(freq=100.0),
                                 block_size=block_size, topk=topk)
    with torch.no_grad():   # non-trivial gate and norm parameters (the initial ones are constants)
        m.gate[0].weight.normal_(0, 0.05)
        if qk_norm:
            for n in (m.q_norm, m.k_norm):
                n.weight.uniform_(0.5, 1.5)
                n.bias.normal_(0, 0.1)
    return m.to(dtype).eval()


def _oracle_out(m, x, xpos, idx):
    sd = {k: v.detach().cpu() for k, v in m.state_dict().items()}
    qn = (sd.get("q_norm.weight"), sd.get("q_norm.bias"), sd.get("k_norm.weight"), sd.get("k_norm.bias"))
    return oracle.sparse_layer(x, sd["qkv.weight"], sd.get("qkv.bias"), sd["gate.0.weight"], sd["gate.0.bias"],
                               sd["proj.weight"], sd.get("proj.bias"), m.num_heads, m.block_size ** 2, m.topk,
                               xpos=xpos, qn_w=qn[0], qn_b=qn[1], kn_w=qn[2], kn_b=qn[3], idx_override=idx)


@pytest.mark.parametrize("dtype,tol", [(torch.bfloat16, 4e-2), (torch.float32, 2e-4)])
@pytest.mark.parametrize("n,block_size,topk", [(320, 8, 2), (200, 8, 4), (160, 4, 4), (64, 8, 1), (1100, 16, 2)])
def test_layer_matches_the_oracle(dtype, tol, n, block_size, topk):
    b, dim, heads = 2, 128, 2
    m = _make(dim, heads, block_size, topk, dtype, seed=n)
    g = torch.Generator().manual_seed(n + 1)
    x = torch.randn((b, n, dim), generator=g).to(dtype)
    side = 24
    xpos = torch.stack((torch.arange(n) // side, torch.arange(n) % side), dim=-1)[None].expand(b, n, 2).contiguous()
    m.keep_topk_idx = True
    with torch.no_grad():
        got = m.to(DEV)(x.to(DEV), xpos=xpos.to(DEV))
    idx = m.last_topk_idx.cpu()
    m.cpu()
    ref_own = _oracle_out(m, x, xpos, None)                     # the oracle's own block choice
    ref = _oracle_out(m, x, xpos, idx)                          # the oracle on the module's block choice
    assert got.shape == (b, n, dim) and got.dtype == dtype
    assert max_abs(got, ref["out"].float()) <= tol
    agree = (idx == ref_own["idx"]).float().mean().item()
    assert agree >= (0.9 if dtype == torch.bfloat16 else 0.99), agree


def test_layer_without_norm_and_positions():
    b, n, dim, heads = 1, 256, 128, 2
    m = _make(dim, heads, 8, 2, torch.bfloat16, seed=5, qk_norm=False)
    x = torch.randn((b, n, dim), generator=torch.Generator().manual_seed(6)).to(torch.bfloat16)
    m.keep_topk_idx = True
    with torch.no_grad():
        got = m.to(DEV)(x.to(DEV))
    idx = m.last_topk_idx.cpu()
    ref = _oracle_out(m.cpu(), x, None, idx)
    assert max_abs(got, ref["out"].float()) <= 4e-2


def test_layer_refuses_gradients_where_no_backward_kernel_is_built():
    m = _make(128, 2, 2, 2, torch.bfloat16, seed=7).to(DEV)      # block 4: the backward kernels are built for blocks 64 and 16
    x = torch.randn((1, 128, 128), device=DEV, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError):
        m(x)                      # parameters require grad and grad mode is on
    with torch.no_grad():
        assert m(x).shape == x.shape


# ------------------------------------------------------------------------------------ fused qk-norm + RoPE kernel
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("with_norm,with_pos", [(True, True), (True, False), (False, True)])
def test_norm_rope_kernel_matches_the_torch_modules(dtype, with_norm, with_pos):
    """One pass of LayerNorm(64) + cast + RoPE2D against the separate torch modules on the same device, for a strided
    view of a packed projection.  Same rounding points; the LayerNorm reduction order differs, so a few values may
    land on the neighbouring representable number."""
    import speed3r_amd as s3r
    b, h, n, d = 2, 3, 333, 64
    g = torch.Generator().manual_seed(11)
    qkv = torch.randn((b, n, 3 * h * d), generator=g).to(dtype).to(DEV)
    x = qkv.view(b, n, 3, h, d).permute(2, 0, 3, 1, 4)[1]                      # k as a strided [B,H,N,D] view
    pos = torch.randint(0, 41, (b, n, 2), generator=g).to(DEV)
    rope = RoPE2D(freq=100.0)
    ln = torch.nn.LayerNorm(d, eps=1e-6).to(DEV)
    with torch.no_grad():
        ln.weight.uniform_(0.5, 1.5)
        ln.bias.normal_(0, 0.1)
    ln = ln.to(dtype)
    cos, sin = rope.tables(d, 41, DEV, dtype)
    with torch.no_grad():
        got = s3r.sparse_attn.ops.norm_rope(x, pos if with_pos else None, cos if with_pos else None, sin if with_pos else None,
                                            ln.weight if with_norm else None, ln.bias if with_norm else None, 1e-6)
        want = ln(x).to(dtype) if with_norm else x
        want = rope(want, pos) if with_pos else want
    assert got.shape == (b, h, n, d) and got.is_contiguous()
    tol = {torch.bfloat16: 4e-2, torch.float16: 5e-3, torch.float32: 1e-5}[dtype]
    assert max_abs(got, want.float()) <= tol
    if not with_norm:
        assert torch.equal(got, want)                                              # no reduction involved: bit-identical
    elif dtype != torch.float32:
        assert (got == want).float().mean().item() >= 0.97


@pytest.mark.parametrize("n,block_size,topk", [(320, 8, 2), (200, 8, 2), (320, 4, 4), (200, 4, 4)])
def test_layer_gradients_match_autograd_through_the_oracle(n, block_size, topk):
    b, dim, heads = 1, 128, 2
    m = _make(dim, heads, block_size, topk, torch.bfloat16, seed=40 + n)
    g = torch.Generator().manual_seed(41 + n)
    x = torch.randn((b, n, dim), generator=g).to(torch.bfloat16)
    gout = torch.randn((b, n, dim), generator=g).to(torch.bfloat16)
    side = 24
    xpos = torch.stack((torch.arange(n) // side, torch.arange(n) % side), dim=-1)[None].expand(b, n, 2).contiguous()
    m.to(DEV).train()
    m.keep_topk_idx = True
    xd = x.to(DEV).requires_grad_(True)
    out = m(xd, xpos=xpos.to(DEV))
    with torch.no_grad():
        m.eval()
        ref_fwd = m(x.to(DEV), xpos=xpos.to(DEV))        # the inference path (fused kernels) on the same weights
        m.train()
    assert max_abs(out.detach(), ref_fwd) <= 4e-2
    out.backward(gout.to(DEV))
    idx = m.last_topk_idx.cpu()
    got = {k: p.grad.detach().float().cpu() for k, p in m.named_parameters() if p.grad is not None}
    got["x"] = xd.grad.detach().float().cpu()
    # the oracle in fp32 on the same (bf16-rounded) parameters and the module's block choice
    m.cpu()
    params = {k: v.detach().float().requires_grad_(True) for k, v in m.state_dict().items()}
    xr = x.float().requires_grad_(True)
    ref = oracle.sparse_layer(xr, params["qkv.weight"], params.get("qkv.bias"), params["gate.0.weight"], params["gate.0.bias"],
                              params["proj.weight"], params.get("proj.bias"), heads, block_size ** 2, topk, xpos=xpos,
                              qn_w=params.get("q_norm.weight"), qn_b=params.get("q_norm.bias"),
                              kn_w=params.get("k_norm.weight"), kn_b=params.get("k_norm.bias"), idx_override=idx)
    ref["out"].backward(gout.float())
    want = {k: v.grad for k, v in params.items() if v.grad is not None}
    want["x"] = xr.grad
    assert set(want) == set(got), (sorted(want), sorted(got))
    for k in want:
        tol = 5e-2 * max(1.0, float(want[k].abs().max()))
        assert max_abs(got[k], want[k]) <= tol, (k, max_abs(got[k], want[k]), tol)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("n,block,with_norm,with_pos", [(320, 64, True, True), (200, 64, True, True), (1041, 16, True, True),
                                                        (77, 16, False, True), (130, 64, True, False), (5, 64, True, True)])
@pytest.mark.parametrize("k_bias", [False, True])
def test_one_pass_over_the_packed_projection_equals_pooling_then_norm_rope(dtype, n, block, with_norm, with_pos, k_bias):
    """s3r_qkv_prepass (block means of raw q, k, v + LayerNorm + RoPE of q and k in one pass) against s3r_pool_mean on
    the packed projection followed by s3r_norm_rope on q and k: the same bits, ragged last blocks included.  With both
    LayerNorm biases and positions (``k_bias``) the kernel runs the instance the layer module launches, in which norm,
    biases and rotation are compile-time facts; without the k bias the general one."""
    from speed3r_amd.sparse_attn import ops
    b, h = 2, 3
    g = torch.Generator().manual_seed(n + block)
    qkv = (torch.randn((b, n, 3 * h * 64), generator=g) * 0.7).to(dtype).to(DEV)
    pos = torch.randint(0, 40, (b, n, 2), generator=g).to(DEV) if with_pos else None
    rope = RoPE2D(freq=100.0)
    cos, sin = rope.tables(64, 40, DEV, dtype) if with_pos else (None, None)
    lnq = ((1 + 0.3 * torch.randn(64, generator=g)).to(dtype).to(DEV), (0.2 * torch.randn(64, generator=g)).to(dtype).to(DEV))
    lnk = ((1 + 0.3 * torch.randn(64, generator=g)).to(dtype).to(DEV),
           (0.2 * torch.randn(64, generator=g)).to(dtype).to(DEV) if k_bias else None)
    got = ops.qkv_prepass(qkv, h, block, pos, cos, sin, lnq if with_norm else None, lnk if with_norm else None, 1e-6)
    q, k, v = qkv.view(b, n, 3, h, 64).permute(2, 0, 3, 1, 4).unbind(0)
    want_c = ops.pool_qkv_packed(qkv, h, block)
    want_q = ops.norm_rope(q, pos, cos, sin, lnq[0] if with_norm else None, lnq[1] if with_norm else None, 1e-6)
    want_k = ops.norm_rope(k, pos, cos, sin, lnk[0] if with_norm else None, lnk[1] if with_norm else None, 1e-6)
    assert torch.equal(got[0], want_q) and torch.equal(got[1], want_k)
    assert got[2].data_ptr() == v.data_ptr() and got[2].stride() == v.stride()
    for a, w in zip(got[3:], want_c):
        assert a.shape == (b, h, -(-n // block), 64) and torch.equal(a, w)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows", [165, 166, 400])
def test_one_pass_with_rotation_tables_around_the_lds_limit(dtype, rows):
    """The layer's instance keeps fp32 copies of the rotation tables in LDS while three tables of ``rows`` x 16 values
    and the LayerNorm rows fit 32 KB (165 rows do, 166 do not); beyond that it reads the caller's tables as before.
    Both sides of the limit give the bits of pooling followed by s3r_norm_rope, positions up to the last row included."""
    from speed3r_amd.sparse_attn import ops
    b, h, n, block = 1, 2, 700, 64
    g = torch.Generator().manual_seed(rows)
    qkv = (torch.randn((b, n, 3 * h * 64), generator=g) * 0.7).to(dtype).to(DEV)
    pos = torch.randint(0, rows, (b, n, 2), generator=g)
    pos[0, :4] = torch.tensor([[0, rows - 1], [rows - 1, 0], [rows - 1, rows - 1], [0, 0]])
    pos = pos.to(DEV)
    cos, sin = RoPE2D(freq=100.0).tables(64, rows, DEV, dtype)
    ln = [((1 + 0.3 * torch.randn(64, generator=g)).to(dtype).to(DEV), (0.2 * torch.randn(64, generator=g)).to(dtype).to(DEV))
          for _ in range(2)]
    got = ops.qkv_prepass(qkv, h, block, pos, cos, sin, ln[0], ln[1], 1e-6)
    q, k, v = qkv.view(b, n, 3, h, 64).permute(2, 0, 3, 1, 4).unbind(0)
    assert torch.equal(got[0], ops.norm_rope(q, pos, cos, sin, ln[0][0], ln[0][1], 1e-6))
    assert torch.equal(got[1], ops.norm_rope(k, pos, cos, sin, ln[1][0], ln[1][1], 1e-6))
    for a, w in zip(got[3:], ops.pool_qkv_packed(qkv, h, block)):
        assert torch.equal(a, w)


def test_one_pass_at_the_headline_token_count_beyond_4_gib_of_offsets():
    """266 496 tokens x 16 heads: the packed projection is 1.6 GB, byte offsets of its rows pass 2^31 (64-bit address
    arithmetic in both routes), the rotated q and k are larger than the last-level cache.  Same bits as pooling followed
    by s3r_norm_rope; the last rows of the last head are also compared with the torch modules."""
    from speed3r_amd.sparse_attn import ops
    b, h, n, block = 1, 16, 266496, 64
    g = torch.Generator(device=DEV).manual_seed(5)
    qkv = (torch.randn((b, n, 3 * h * 64), generator=g, device=DEV, dtype=torch.float32) * 0.7).to(torch.bfloat16)
    t = torch.arange(n, device=DEV) % 1041
    pos = torch.stack((t // 28, t % 28), dim=-1)[None].contiguous()
    rope = RoPE2D(freq=100.0)
    cos, sin = rope.tables(64, 38, DEV, torch.bfloat16)
    gc = torch.Generator().manual_seed(6)
    ln = [((1 + 0.3 * torch.randn(64, generator=gc)).to(torch.bfloat16).to(DEV), (0.2 * torch.randn(64, generator=gc)).to(torch.bfloat16).to(DEV))
          for _ in range(2)]
    got = ops.qkv_prepass(qkv, h, block, pos, cos, sin, ln[0], ln[1], 1e-6)
    q, k, v = qkv.view(b, n, 3, h, 64).permute(2, 0, 3, 1, 4).unbind(0)
    want_q = ops.norm_rope(q, pos, cos, sin, ln[0][0], ln[0][1], 1e-6)
    assert torch.equal(got[0], want_q)
    del want_q
    want_k = ops.norm_rope(k, pos, cos, sin, ln[1][0], ln[1][1], 1e-6)
    assert torch.equal(got[1], want_k)
    del want_k
    for a, w in zip(got[3:], ops.pool_qkv_packed(qkv, h, block)):
        assert torch.equal(a, w)
    # the far end against the eager modules (LayerNorm in fp32 on the bf16 values, rounded, then RoPE2D)
    tail = slice(n - 2082, n)
    lnq = torch.nn.LayerNorm(64, eps=1e-6).to(DEV).to(torch.bfloat16)
    with torch.no_grad():
        lnq.weight.copy_(ln[0][0]); lnq.bias.copy_(ln[0][1])
        want = rope(lnq(q[:, -1:, tail]).to(torch.bfloat16), pos[:, tail])
    assert max_abs(got[0][:, -1:, tail], want.float()) <= 4e-2
    assert (got[0][:, -1:, tail] == want).float().mean().item() >= 0.97


def test_layer_takes_the_one_pass_route_where_it_is_built():
    torch.manual_seed(11)
    m = SparseFlashAttentionRope(dim=128, num_heads=2, qkv_bias=True, qk_norm=True, rope=RoPE2D(100.0), block_size=8, topk=2)
    m = m.to(torch.bfloat16).to(DEV).eval()
    x = torch.randn(1, 200, 128, device=DEV).to(torch.bfloat16)
    pos = torch.randint(0, 30, (1, 200, 2), device=DEV)
    with torch.no_grad():
        m(x, xpos=pos)
        assert m.last_prepass is True and m.last_path == "fused-merge"
        m2 = SparseFlashAttentionRope(dim=128, num_heads=2, block_size=8, topk=2).to(torch.bfloat16).to(DEV).eval()
        m2(x)                                   # no norm, no positions: nothing to do to q and k, no pre-pass
        assert m2.last_prepass is False
        m3 = SparseFlashAttentionRope(dim=128, num_heads=2, qk_norm=True, rope=RoPE2D(100.0), block_size=4, topk=4).to(torch.bfloat16).to(DEV).eval()
        m3(x, xpos=pos)                         # 16-token blocks: separate kernels, the index kernel starts earlier
        assert m3.last_prepass is False and m3.last_path == "fused-merge"
