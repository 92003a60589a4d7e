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
