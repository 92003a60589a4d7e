"""Pins of the layer-level oracle (RoPE2D, block positions) and CPU-side checks of the layer module:
its own RoPE2D against the oracle's, its parameter names and constructor signature."""
import inspect
import math

import pytest
import torch

import oracle
from speed3r_amd.layers import RoPE2D, SparseFlashAttentionRope, block_positions


def _tokens(b, h, n, d, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return torch.randn((b, h, n, d), generator=g).to(dtype)


def _positions(b, n, seed, hi=37):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, hi, (b, n, 2), generator=g)


def test_rope_head_dim_4_is_a_plane_rotation_by_the_coordinate():
    # head_dim 4: y half = dims (0,1), x half = dims (2,3); one frequency, base**0 = 1 -> angle = coordinate in radians
    t = _tokens(1, 1, 5, 4, 0)
    pos = torch.tensor([[[0, 0], [1, 0], [0, 2], [3, 5], [7, 1]]])
    got = oracle.rope2d(t, pos)
    for n in range(5):
        for half, coord in ((0, pos[0, n, 0].item()), (1, pos[0, n, 1].item())):
            a, b = t[0, 0, n, 2 * half].item(), t[0, 0, n, 2 * half + 1].item()
            c, s = math.cos(coord), math.sin(coord)
            assert got[0, 0, n, 2 * half].item() == pytest.approx(a * c - b * s, abs=1e-5)
            assert got[0, 0, n, 2 * half + 1].item() == pytest.approx(b * c + a * s, abs=1e-5)


def test_rope_against_a_complex_number_formulation_fp64():
    b, h, n, d = 2, 3, 17, 64
    t = _tokens(b, h, n, d, 1, torch.float64)
    pos = _positions(b, n, 2)
    got = oracle.rope2d(t, pos, base=100.0)
    quarter = d // 4
    freq = 100.0 ** (-torch.arange(quarter, dtype=torch.float64) / quarter)      # base ** (-2i / (D/2))
    want = torch.empty_like(t)
    for half in range(2):
        blk = t[..., half * d // 2:(half + 1) * d // 2]
        z = torch.complex(blk[..., :quarter], blk[..., quarter:])                  # element j pairs with j + D/4
        ang = pos[..., half].to(torch.float64)[:, None, :, None] * freq
        z = z * torch.polar(torch.ones_like(ang), ang)
        want[..., half * d // 2:half * d // 2 + quarter] = z.real
        want[..., half * d // 2 + quarter:(half + 1) * d // 2] = z.imag
    assert torch.allclose(got, want, atol=2e-5)          # the oracle builds its angle table in fp32, like the reference


def test_rope_invariants():
    b, h, n, d = 1, 2, 9, 32
    q, k = _tokens(b, h, n, d, 3, torch.float64), _tokens(b, h, n, d, 4, torch.float64)
    zero = torch.zeros((b, n, 2), dtype=torch.long)
    assert torch.equal(oracle.rope2d(q, zero), q)                                  # position 0: identity
    pos = _positions(b, n, 5)
    rq = oracle.rope2d(q, pos)
    assert torch.allclose(rq.norm(dim=-1), q.norm(dim=-1), atol=1e-6)              # rotations preserve norms
    moved = pos.clone()
    moved[..., 1] += 11                                                            # x changes: the y half must not
    assert torch.equal(oracle.rope2d(q, moved)[..., :d // 2], rq[..., :d // 2])
    shift = torch.tensor([4, 9])
    dots = torch.einsum("bhnd,bhmd->bhnm", rq, oracle.rope2d(k, pos))
    dots_shifted = torch.einsum("bhnd,bhmd->bhnm", oracle.rope2d(q, pos + shift), oracle.rope2d(k, pos + shift))
    assert torch.allclose(dots, dots_shifted, atol=1e-3)                           # only position differences matter


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_module_rope_equals_oracle_rope(dtype):
    t = _tokens(2, 4, 50, 64, 6, dtype)
    pos = _positions(2, 50, 7)
    assert torch.equal(RoPE2D(freq=100.0)(t, pos), oracle.rope2d(t, pos, base=100.0))


def test_block_positions_known_answers():
    xpos = torch.tensor([[[0, 0], [0, 1], [0, 2], [0, 3], [1, 0], [1, 1], [1, 2], [1, 3], [5, 7], [6, 7]]])
    want = torch.tensor([[[0, 1], [1, 1], [5, 7]]], dtype=torch.int32)             # means (0,1.5)->(0,1), (1,1.5)->(1,1), (5.5,7)->(5,7)
    assert torch.equal(oracle.block_positions(xpos, 4), want)
    assert torch.equal(block_positions(xpos, 4), want)
    xpos2 = _positions(2, 128, 8, hi=50)
    assert torch.equal(block_positions(xpos2, 16), oracle.block_positions(xpos2, 16))
    assert torch.equal(block_positions(xpos2, 16), xpos2.view(2, 8, 16, 2).float().mean(dim=2).int())


def test_layer_module_has_the_reference_constructor_and_parameter_names():
    names = list(inspect.signature(SparseFlashAttentionRope.__init__).parameters)
    assert names[:12] == ["self", "dim", "num_heads", "qkv_bias", "proj_bias", "attn_drop", "proj_drop", "qk_norm",
                          "norm_layer", "rope", "block_size", "topk"]
    m = SparseFlashAttentionRope(dim=128, num_heads=2, qkv_bias=True, qk_norm=True, block_size=8)
    assert set(m.state_dict()) == {"qkv.weight", "qkv.bias", "proj.weight", "proj.bias", "q_norm.weight", "q_norm.bias",
                                   "k_norm.weight", "k_norm.bias", "gate.0.weight", "gate.0.bias"}
    assert torch.count_nonzero(m.gate[0].weight) == 0
    assert torch.equal(m.gate[0].bias.detach(), torch.tensor([-1.0, 1.0, -1.0, 1.0]))
    sig = inspect.signature(m.forward).parameters
    assert list(sig)[:3] == ["x", "attn_bias", "xpos"]       # the reference's call; anything further is optional
    assert all(p.default is not inspect.Parameter.empty for name, p in sig.items() if name not in ("x",))


def test_layer_module_refuses_cpu_tensors():
    m = SparseFlashAttentionRope(dim=128, num_heads=2, block_size=8, topk=2)
    with torch.no_grad(), pytest.raises(Exception):
        m(torch.zeros((1, 128, 128)))


def test_patch_embedding_as_one_gemm_equals_the_convolution():
    """The model's patch embedding (unfold + linear on the Conv2d's parameters) against F.conv2d, fp32 on the CPU."""
    import torch.nn.functional as F
    from speed3r_amd.model.pi3_sparse_like import PatchEncoder
    torch.manual_seed(0)
    enc = PatchEncoder(dim=32, depth=0, num_heads=2, patch=14, grid=(3, 2), num_register=4)
    imgs = torch.rand(2, 3, 45, 31)                       # not multiples of 14: the convolution drops the remainder
    want = F.conv2d(imgs, enc.patch_embed.weight, enc.patch_embed.bias, stride=14).flatten(2).transpose(1, 2)
    got = enc(imgs)                                       # depth 0: tokens = norm(embedding + position) without cls/registers
    f, gh, gw = 2, 3, 2
    x = torch.cat((enc.cls_token.expand(f, -1, -1), want), dim=1) + enc._pos(gh, gw)
    assert torch.allclose(got, enc.norm(x)[:, 1:], atol=1e-5)
