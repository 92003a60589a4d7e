"""The model restatement (``oracle.pi3_sparse_like_forward``: library routines on a state dict) against the package's
model modules on the CPU in fp32.  The package's global blocks need the GPU, so here their attention is replaced by
``oracle.sparse_layer`` on the module's own parameters: what is compared is everything AROUND the sparse layer (patch
embedding, token layout and positions, pre-norm blocks with LayerScale, frame-local attention with qk-norm and RoPE,
head decoders, pixel-shuffle heads, pose head), composed twice independently.  The GPU test of the same name part
(tests/test_gpu_model.py) then runs the real layer and kernels against this restatement."""
import torch

import oracle
from speed3r_amd.model import Pi3SparseLike


def _small_model(seed=0, **kw):
    torch.manual_seed(seed)
    m = Pi3SparseLike(dim=128, enc_depth=2, dec_depth=4, num_heads=2, head_depth=1, block_tokens=16, topk=4,
                      **{"grid": (4, 6), **kw})
    with torch.no_grad():                      # non-trivial values where the constructors put zeros or near-zeros
        for name, p in m.named_parameters():
            if name.endswith("gamma"):
                p.copy_(0.5 + 0.5 * torch.rand_like(p))
            elif "gate.0" in name or name.endswith("cls_token") or name.endswith("register_tokens") or name == "register_token":
                p.copy_(0.3 * torch.randn_like(p))
            elif name.endswith("norm.weight") or name.endswith("norm1.weight") or name.endswith("norm2.weight"):
                p.copy_(1 + 0.2 * torch.randn_like(p))
            elif name.endswith(".bias"):
                p.copy_(0.1 * torch.randn_like(p))
    return m.eval()


def _with_oracle_layers(m):
    """Global blocks' attention -> oracle.sparse_layer on the module's parameters (CPU stand-in for the HIP layer)."""
    for blk in m.global_decoder:
        a = blk.attn

        def fwd(x, attn_bias=None, xpos=None, n_pos=None, a=a):
            return oracle.sparse_layer(x, a.qkv.weight, a.qkv.bias, a.gate[0].weight, a.gate[0].bias, a.proj.weight, a.proj.bias,
                                       a.num_heads, a.block_size ** 2, a.topk, xpos=xpos, qn_w=a.q_norm.weight,
                                       qn_b=a.q_norm.bias, kn_w=a.k_norm.weight, kn_b=a.k_norm.bias, ln_eps=a.q_norm.eps)["out"]
        a.forward = fwd
    return m


def test_restatement_equals_the_modules_around_the_sparse_layer():
    m = _with_oracle_layers(_small_model())
    frames, hh, ww = 6, 56, 84                 # 24 patches + 5 register tokens = 29 tokens per frame: 174 tokens, ragged last block
    imgs = torch.rand((1, frames, 3, hh, ww), generator=torch.Generator().manual_seed(1))
    with torch.no_grad():
        got = m(imgs, return_features=True)
        want = oracle.pi3_sparse_like_forward(m.state_dict(), imgs, heads=2, patch=14, block_tokens=16, topk=4, return_features=True)
    assert set(got) == set(want)
    for key in want:
        assert got[key].shape == want[key].shape, key
        scale = max(1.0, want[key].abs().max().item())
        assert (got[key].float() - want[key]).abs().max().item() <= 2e-4 * scale, key
    rot = want["camera_poses"][0, :, :3, :3].double()
    assert torch.allclose(rot @ rot.transpose(-1, -2), torch.eye(3, dtype=torch.float64).expand(frames, 3, 3), atol=1e-5)


def test_restatement_reacts_to_every_parameter_group():
    """No part of the restatement is dead: perturbing any parameter group changes its features or outputs."""
    m = _small_model(1)
    imgs = torch.rand((1, 3, 3, 56, 84), generator=torch.Generator().manual_seed(2))
    sd = {k: v.clone() for k, v in m.state_dict().items()}
    base = oracle.pi3_sparse_like_forward(sd, imgs, heads=2, patch=14, block_tokens=16, topk=4, return_features=True)
    groups = ["encoder.patch_embed.weight", "encoder.pos_embed", "encoder.blocks.1.mlp.fc2.weight", "register_token",
              "local_decoder.0.attn.q_norm.weight", "local_decoder.1.ls1.gamma", "global_decoder.0.attn.gate.0.bias",
              "global_decoder.1.attn.k_norm.bias", "global_decoder.1.mlp.fc1.weight", "point_decoder.blocks.0.attn.qkv.weight",
              "conf_head.proj.weight", "camera_head.mlp.2.weight", "camera_decoder.linear_out.bias"]
    for name in groups:
        sd2 = dict(sd)
        sd2[name] = sd[name] + 0.05 * torch.randn(sd[name].shape, generator=torch.Generator().manual_seed(3))
        out = oracle.pi3_sparse_like_forward(sd2, imgs, heads=2, patch=14, block_tokens=16, topk=4, return_features=True)
        assert any((out[k] - base[k]).abs().max().item() > 1e-6 for k in base), name


def test_restatement_in_the_reference_token_order():
    """The reference model's own token pipeline (no register tokens, positions from 0, 4 x 4-tile-major order through
    the decoder and row-major order again in front of the heads): the package's modules reorder with reshape/permute,
    the restatement with a gather index built by plain loops.  8 x 8 patches per frame = 4 tiles = four 16-token blocks."""
    m = _with_oracle_layers(_small_model(2, grid=(8, 8), num_register=0, token_order="tile"))
    frames, hh, ww = 3, 112, 112
    imgs = torch.rand((1, frames, 3, hh, ww), generator=torch.Generator().manual_seed(5))
    with torch.no_grad():
        got = m(imgs, return_features=True)
        want = oracle.pi3_sparse_like_forward(m.state_dict(), imgs, heads=2, patch=14, block_tokens=16, topk=4,
                                              return_features=True, tile=4)
        row = oracle.pi3_sparse_like_forward(m.state_dict(), imgs, heads=2, patch=14, block_tokens=16, topk=4, return_features=True)
    for key in want:
        assert got[key].shape == want[key].shape, key
        scale = max(1.0, want[key].abs().max().item())
        assert (got[key].float() - want[key]).abs().max().item() <= 2e-4 * scale, key
    # the order matters: the same weights on row-major tokens (blocks = runs of 16 tokens of a patch row pair) differ
    assert (row["features"] - want["features"]).abs().max().item() > 1e-3
