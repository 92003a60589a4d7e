"""The Pi3_Sparse-style model on the GPU: a small configuration against the CPU restatement of the model
(oracle.pi3_sparse_like_forward, fp32 library routines + the layer oracle), the full-size end-to-end workload once,
and the model's dense attention module against the eager expression."""
import pytest
import torch

import oracle
from speed3r_amd.layers import RoPE2D, SparseFlashAttentionRope
from speed3r_amd.model import Pi3SparseLike

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_small_model_forward_shapes_and_finiteness():
    torch.manual_seed(0)
    m = Pi3SparseLike(dim=128, enc_depth=2, dec_depth=4, num_heads=2, head_depth=1, grid=(4, 6), topk=4)
    assert all(isinstance(b.attn, SparseFlashAttentionRope) for b in m.global_decoder)
    m = m.to(torch.bfloat16).to(DEV).eval()
    frames, hh, ww = 12, 56, 84                      # 4 x 6 patches + 5 register tokens = 29 tokens per frame, 348 in all
    imgs = torch.rand((1, frames, 3, hh, ww), generator=torch.Generator().manual_seed(1)).to(DEV)
    with torch.no_grad():
        out = m(imgs)
    assert out["points"].shape == (1, frames, hh, ww, 3)
    assert out["local_points"].shape == (1, frames, hh, ww, 3)
    assert out["conf"].shape == (1, frames, hh, ww, 1)
    assert out["camera_poses"].shape == (1, frames, 4, 4)
    for v in out.values():
        assert torch.isfinite(v).all()
    rot = out["camera_poses"][0, :, :3, :3].double()
    assert torch.allclose(rot @ rot.transpose(-1, -2), torch.eye(3, dtype=torch.float64, device=DEV).expand(frames, 3, 3), atol=1e-4)


@pytest.mark.parametrize("n,qk_norm", [(29, False), (1041, True), (64, True)])
def test_frame_local_dense_attention_matches_eager_fp32(n, qk_norm):
    """The model's dense attention module (package dense flash kernel writing [B,N,H,D] directly) against the eager
    fp32 expression softmax(q k^T / sqrt(d)) v on the module's own bf16 projections; tolerance 2e-2 (bf16 I/O)."""
    from speed3r_amd.model.pi3_sparse_like import DenseAttentionRope
    torch.manual_seed(2)
    b, h, c = 3, 2, 128
    m = DenseAttentionRope(c, num_heads=h, qk_norm=qk_norm).to(torch.bfloat16).to(DEV).eval()
    x = torch.randn(b, n, c, device=DEV).to(torch.bfloat16)
    with torch.no_grad():
        got = m(x)
        q, k, v = m.qkv(x).view(b, n, 3, h, c // h).permute(2, 0, 3, 1, 4).unbind(0)
        q, k = m.q_norm(q).to(x.dtype), m.k_norm(k).to(x.dtype)
        p = torch.softmax(q.float() @ k.float().transpose(-1, -2) / 8.0, dim=-1)
        o = (p @ v.float()).to(x.dtype)
        want = m.proj(o.transpose(1, 2).reshape(b, n, c))
    assert (got.float() - want.float()).abs().max().item() <= 2e-2


def test_dense_attention_into_a_caller_view():
    """compressed_attn_topk(out=...) writes the [B,H,L,D] result through arbitrary strides of the first three dimensions."""
    from speed3r_amd.sparse_attn import ops
    torch.manual_seed(3)
    b, h, n, d = 2, 3, 150, 64
    q, k, v = ((torch.randn(b, h, n, d, device=DEV) / 2).to(torch.bfloat16) for _ in range(3))
    ref = ops.compressed_attn_topk(q, k, v, None)[0]
    buf = torch.full((b, n, h, d), 7.0, dtype=torch.bfloat16, device=DEV)
    o, _ = ops.compressed_attn_topk(q, k, v, None, out=buf.permute(0, 2, 1, 3))
    assert o.data_ptr() == buf.data_ptr()
    assert torch.equal(buf.permute(0, 2, 1, 3), ref)


def _randomised_small_model(seed=0, **kw):
    torch.manual_seed(seed)
    m = Pi3SparseLike(dim=128, enc_depth=2, dec_depth=4, num_heads=2, head_depth=1, block_tokens=16, topk=4,
                      **{"grid": (4, 6), **kw})
    with torch.no_grad():                      # non-trivial values where the constructors put zeros or near-zeros
        for name, p in m.named_parameters():
            if name.endswith("gamma"):
                p.copy_(0.5 + 0.5 * torch.rand_like(p))
            elif "gate.0" in name or name.endswith("cls_token") or name.endswith("register_tokens") or name == "register_token":
                p.copy_(0.3 * torch.randn_like(p))
            elif name.endswith(".bias"):
                p.copy_(0.1 * torch.randn_like(p))
    return m.eval()


def test_small_model_fp32_matches_the_cpu_restatement():
    """Same weights, same images: the package's forward on the GPU (its layer module and kernels in their fp32
    instances: pooling, norm/RoPE, both attention operators, merge, block norms) against the eager fp32 restatement on
    the CPU.  348 tokens in blocks of 16 with a ragged last block, top-4.  Tolerance 1e-4 of each output's scale
    (accumulation-order differences only, no low-precision rounding anywhere; measured 5e-6)."""
    m = _randomised_small_model()
    frames, hh, ww = 12, 56, 84
    imgs = torch.rand((1, frames, 3, hh, ww), generator=torch.Generator().manual_seed(1))
    want = oracle.pi3_sparse_like_forward(m.state_dict(), imgs, heads=2, patch=14, block_tokens=16, topk=4, return_features=True)
    m = m.to(DEV)
    with torch.no_grad():
        got = m(imgs.to(DEV), return_features=True)
    assert all(b.attn.last_path in ("fused-merge", "two-operators") for b in m.global_decoder)
    for key in want:
        scale = max(1.0, want[key].abs().max().item())
        err = (got[key].float().cpu() - want[key]).abs().max().item()
        assert err <= 1e-4 * scale, (key, err, scale)


def test_small_model_bf16_stays_close_to_the_fp32_restatement():
    """The bf16 model (fused kernels: packed pooling, norm/RoPE, index kernel, selection with the merge in its
    epilogue, dense flash attention, block norms) against the fp32 restatement on the bf16-rounded weights.  bf16
    carries 8 bits and a near-tie in a block selection may go the other way, so the bar is statistical: relative L2
    error of the decoder features and of every output at most 2 % (measured 0.3-0.7 %)."""
    m = _randomised_small_model(3).to(torch.bfloat16)
    frames, hh, ww = 12, 56, 84
    imgs = torch.rand((1, frames, 3, hh, ww), generator=torch.Generator().manual_seed(4))
    want = oracle.pi3_sparse_like_forward(m.state_dict(), imgs, heads=2, patch=14, block_tokens=16, topk=4, return_features=True)
    m = m.to(DEV)
    with torch.no_grad():
        got = m(imgs.to(DEV), return_features=True)
    assert all(b.attn.last_path == "fused-merge" for b in m.global_decoder)
    for key, bar in (("features", 0.02), ("local_points", 0.02), ("points", 0.02), ("conf", 0.02), ("camera_poses", 0.02)):
        g, w = got[key].float().cpu(), want[key]
        rel = ((g - w).norm() / w.norm()).item()
        assert rel <= bar, (key, rel)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_small_model_in_the_reference_token_order(dtype):
    """The reference model's own setting in small: no register tokens, positions from 0, 4 x 4-tile-major token order
    through the decoder (pi3_sparse.py:29-71,228-229,265-269), 16-token blocks = one tile each, against the restatement
    extended the same way (a gather index built by plain loops).  12 frames of 8 x 12 patches = 1152 tokens = 72 blocks,
    top-8.  fp32: 1e-4 of each output's scale; bf16: relative L2 error at most 2 % (near-ties in a selection may flip)."""
    torch.manual_seed(6)
    m = Pi3SparseLike(dim=128, enc_depth=2, dec_depth=4, num_heads=2, head_depth=1, grid=(8, 12), block_tokens=16, topk=8,
                      num_register=0, token_order="tile")
    with torch.no_grad():
        for name, p in m.named_parameters():
            if name.endswith("gamma"):
                p.copy_(0.5 + 0.5 * torch.rand_like(p))
            elif "gate.0" in name or name.endswith("cls_token") or name.endswith("register_tokens"):
                p.copy_(0.3 * torch.randn_like(p))
            elif name.endswith(".bias"):
                p.copy_(0.1 * torch.randn_like(p))
    m = m.eval().to(dtype)
    frames, hh, ww = 12, 112, 168
    imgs = torch.rand((1, frames, 3, hh, ww), generator=torch.Generator().manual_seed(7))
    want = oracle.pi3_sparse_like_forward(m.state_dict(), imgs, heads=2, patch=14, block_tokens=16, topk=8,
                                          return_features=True, tile=4)
    m = m.to(DEV)
    with torch.no_grad():
        got = m(imgs.to(DEV), return_features=True)
    assert all(b.attn.last_path in ("fused-merge", "two-operators") for b in m.global_decoder)
    for key in want:
        g, w = got[key].float().cpu(), want[key]
        if dtype == torch.float32:
            assert (g - w).abs().max().item() <= 1e-4 * max(1.0, w.abs().max().item()), key
        else:
            assert ((g - w).norm() / w.norm()).item() <= 0.02, key


def test_rope_tables_follow_the_frame_size(monkeypatch):
    """Frames larger than the grid the model was built for: the fused norm/RoPE kernel's tables are sized from the
    call (positions beyond a table would be clamped): the model's dense attention with RoPE on a 45-wide position range
    against the torch RoPE2D module."""
    from speed3r_amd.model.pi3_sparse_like import DenseAttentionRope
    torch.manual_seed(5)
    rope = RoPE2D(freq=100.0, max_positions=0)
    a = DenseAttentionRope(128, num_heads=2, qk_norm=True, rope=rope).to(torch.bfloat16).to(DEV).eval()
    n = 200
    pos = torch.stack((torch.arange(n) % 45, torch.arange(n) // 5), dim=-1)[None].to(DEV)
    x = torch.randn(1, n, 128, device=DEV).to(torch.bfloat16)
    with torch.no_grad():
        got = a(x, xpos=pos)
        q, k, v = a.qkv(x).view(1, n, 3, 2, 64).permute(2, 0, 3, 1, 4).unbind(0)
        q, k = rope(a.q_norm(q).to(x.dtype), pos), rope(a.k_norm(k).to(x.dtype), pos)
        p = torch.softmax(q.float() @ k.float().transpose(-1, -2) / 8.0, dim=-1)
        want = a.proj((p @ v.float()).to(x.dtype).transpose(1, 2).reshape(1, n, 128))
    assert (got.float() - want.float()).abs().max().item() <= 2e-2
    m = Pi3SparseLike(dim=128, enc_depth=1, dec_depth=2, num_heads=2, head_depth=1, grid=(4, 6), topk=4).to(torch.bfloat16).to(DEV).eval()
    imgs = torch.rand((1, 2, 3, 14 * 9, 14 * 41), device=DEV)          # 9 x 41 patches on a model built for 4 x 6
    from speed3r_amd.sparse_attn import ops
    rows = []
    real_nr, real_pp = ops.norm_rope, ops.qkv_prepass
    monkeypatch.setattr(ops, "norm_rope", lambda x, pos, cos, sin, *a, **k: (rows.append(None if cos is None else cos.shape[0]), real_nr(x, pos, cos, sin, *a, **k))[1])
    monkeypatch.setattr(ops, "qkv_prepass", lambda qkv, h, blk, pos, cos, sin, *a, **k: (rows.append(None if cos is None else cos.shape[0]), real_pp(qkv, h, blk, pos, cos, sin, *a, **k))[1])
    with torch.no_grad():
        m(imgs)
    assert rows and all(r in (None, 42) for r in rows) and 42 in rows   # every rotating kernel got a table for coordinates 0..41
    assert m.rope.max_positions == 8          # as constructed (grid 4 x 6): the call's table size travels with the call


def test_end_to_end_workload_100_frames_518x392():
    """The end-to-end configuration itself, once: 100 frames of 518x392 (104 100 tokens), ViT-L/14 encoder, 36-layer
    decoder, heads, random-init bf16, seed 4.  Shapes, finiteness, orthonormal rotations, and every one of the 18
    global blocks on the fused route (packed pooling, index kernel, selection with the merge in its epilogue)."""
    torch.manual_seed(4)
    with torch.device(DEV):
        m = Pi3SparseLike()
    m = m.to(torch.bfloat16).eval()
    frames = 100
    imgs = torch.rand((1, frames, 3, 518, 392), generator=torch.Generator().manual_seed(4)).to(DEV)
    with torch.no_grad():
        out = m(imgs)
    torch.cuda.synchronize()
    assert len(m.global_decoder) == 18 and all(b.attn.last_path == "fused-merge" for b in m.global_decoder)
    assert out["points"].shape == (1, frames, 518, 392, 3) and out["conf"].shape == (1, frames, 518, 392, 1)
    assert out["camera_poses"].shape == (1, frames, 4, 4)
    for v in out.values():
        assert torch.isfinite(v).all()
    rot = out["camera_poses"][0, :, :3, :3].double()
    assert torch.allclose(rot @ rot.transpose(-1, -2), torch.eye(3, dtype=torch.float64, device=DEV).expand(frames, 3, 3), atol=1e-4)
    del m, out
    torch.cuda.empty_cache()


def test_end_to_end_workload_in_the_reference_setting_100_frames_504x392():
    """The reference model's own setting at full size, once: 100 frames of 504 x 392 (a multiple of 56: 36 x 28 patches
    = 63 tiles of 4 x 4, 100 800 tokens), no register tokens, tile-major order, 16-token blocks, top-32
    (sparse_attention.py:73,98,112).  Shapes, finiteness, orthonormal rotations, all 18 global blocks on the fused route."""
    torch.manual_seed(4)
    with torch.device(DEV):
        m = Pi3SparseLike(grid=(36, 28), num_register=0, token_order="tile", block_tokens=16, topk=32)
    m = m.to(torch.bfloat16).eval()
    frames = 100
    imgs = torch.rand((1, frames, 3, 504, 392), generator=torch.Generator().manual_seed(4)).to(DEV)
    with torch.no_grad():
        out = m(imgs)
    torch.cuda.synchronize()
    assert len(m.global_decoder) == 18 and all(b.attn.last_path == "fused-merge" for b in m.global_decoder)
    assert out["points"].shape == (1, frames, 504, 392, 3) and out["camera_poses"].shape == (1, frames, 4, 4)
    for v in out.values():
        assert torch.isfinite(v).all()
    rot = out["camera_poses"][0, :, :3, :3].double()
    assert torch.allclose(rot @ rot.transpose(-1, -2), torch.eye(3, dtype=torch.float64, device=DEV).expand(frames, 3, 3), atol=1e-4)
    del m, out
    torch.cuda.empty_cache()
