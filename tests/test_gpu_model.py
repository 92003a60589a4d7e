"""The Pi3_Sparse-style model runs end to end on the GPU (small configuration) and its global blocks use the sparse layer."""
import pytest
import torch

from speed3r_amd.layers import SparseFlashAttentionRope
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
