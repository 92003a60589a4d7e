"""CPU restatement, in eager fp32 torch, of the Pi3_Sparse-style model that ``speed3r_amd.model`` builds for the
end-to-end figure.

TEST INFRASTRUCTURE ONLY -- never imported by the product package.

The model follows the reference's structure (pi3/models/pi3_sparse.py:214-321: encoder -> alternating frame-local /
global decoder blocks -> point, confidence and camera decoders and heads; pi3/models/layers/block.py:259-335: pre-norm
block with LayerScale; pi3/models/layers/attention.py:324-348: dense attention with qk-norm and RoPE) with the Pi3
teacher's token layout (register tokens, then patches in row-major order) or, with ``tile > 0``, with the reference
model's own one (no register tokens, positions from 0, patches of a frame in tile-major order through the decoder and
back in row-major order in front of the heads: pi3_sparse.py:29-71,163-169,228-229,265-269).  Here every piece is a library routine on
the parameters of a ``state_dict``: ``F.conv2d`` for the patch embedding, ``F.layer_norm``, ``F.linear``, ``F.gelu``,
``F.scaled_dot_product_attention`` for the frame-local attentions, ``rope2d`` and ``sparse_layer`` of this package
(both pinned on their own) for the rotary embedding and the global blocks, ``F.pixel_shuffle`` for the dense heads.
Nothing of ``speed3r_amd`` is used: the restatement reads parameter NAMES only.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F

from .sparse_layer_oracle import rope2d, sparse_layer

LN_EPS = 1e-6


def _ln(x, sd, name):
    return F.layer_norm(x, (x.shape[-1],), sd[name + ".weight"], sd[name + ".bias"], LN_EPS)


def _dense_attention(x, sd, pre, heads, pos, qk_norm, rope_base):
    b, n, c = x.shape
    d = c // heads
    qkv = F.linear(x, sd[pre + ".qkv.weight"], sd[pre + ".qkv.bias"]).reshape(b, n, 3, heads, d).permute(2, 0, 3, 1, 4)
    q, k, v = qkv[0], qkv[1], qkv[2]
    if qk_norm:
        q = F.layer_norm(q, (d,), sd[pre + ".q_norm.weight"], sd[pre + ".q_norm.bias"], LN_EPS)
        k = F.layer_norm(k, (d,), sd[pre + ".k_norm.weight"], sd[pre + ".k_norm.bias"], LN_EPS)
    if pos is not None:
        q, k = rope2d(q, pos, rope_base), rope2d(k, pos, rope_base)
    o = F.scaled_dot_product_attention(q, k, v).transpose(1, 2).reshape(b, n, c)
    return F.linear(o, sd[pre + ".proj.weight"], sd[pre + ".proj.bias"])


def _block(x, sd, pre, attn, layer_scale):
    a = attn(_ln(x, sd, pre + ".norm1"))
    x = x + (sd[pre + ".ls1.gamma"] * a if layer_scale else a)
    m = F.linear(F.gelu(F.linear(_ln(x, sd, pre + ".norm2"), sd[pre + ".mlp.fc1.weight"], sd[pre + ".mlp.fc1.bias"])),
                 sd[pre + ".mlp.fc2.weight"], sd[pre + ".mlp.fc2.bias"])
    return x + (sd[pre + ".ls2.gamma"] * m if layer_scale else m)


def _count(sd, prefix):
    return 1 + max(int(k[len(prefix):].split(".")[0]) for k in sd if k.startswith(prefix))


def tile_major_index(gh: int, gw: int, tile: int) -> torch.Tensor:
    """``perm[i]`` = row-major index of the token that stands at place ``i`` of the tile-major order: place
    ``((ty * (gw // tile) + tx) * tile + py) * tile + px`` holds token ``(ty * tile + py, tx * tile + px)``
    (pi3_sparse.py:29-45, 'b (nh ph) (nw pw) d -> b (nh nw ph pw) d')."""
    perm = torch.empty(gh * gw, dtype=torch.long)
    i = 0
    for ty in range(gh // tile):
        for tx in range(gw // tile):
            for py in range(tile):
                for px in range(tile):
                    perm[i] = (ty * tile + py) * gw + tx * tile + px
                    i += 1
    return perm


def pi3_sparse_like_forward(sd: dict, imgs: torch.Tensor, heads: int, patch: int, block_tokens: int, topk: int,
                            rope_base: float = 100.0, return_features: bool = False, tile: int = 0) -> dict:
    """imgs ``[B,F,3,H,W]`` in [0,1], ``sd`` the model's state dict as fp32 CPU tensors -> the model's outputs.
    ``tile > 0``: the reference model's token pipeline (no register tokens allowed in ``sd``)."""
    sd = {k: v.detach().float().cpu() for k, v in sd.items()}
    b, f, _, hh, ww = imgs.shape
    gh, gw = hh // patch, ww // patch
    dim = sd["register_token"].shape[-1]
    x = ((imgs.float() - sd["image_mean"]) / sd["image_std"]).reshape(b * f, 3, hh, ww)
    # encoder: patch embedding, class token, learned positions, register tokens, dense blocks without RoPE
    x = F.conv2d(x, sd["encoder.patch_embed.weight"], sd["encoder.patch_embed.bias"], stride=patch).flatten(2).transpose(1, 2)
    x = torch.cat((sd["encoder.cls_token"].expand(b * f, -1, -1), x), dim=1) + sd["encoder.pos_embed"]
    nreg_enc = sd["encoder.register_tokens"].shape[1]
    x = torch.cat((x[:, :1], sd["encoder.register_tokens"].expand(b * f, -1, -1), x[:, 1:]), dim=1)
    for i in range(_count(sd, "encoder.blocks.")):
        pre = f"encoder.blocks.{i}"
        x = _block(x, sd, pre, lambda y: _dense_attention(y, sd, pre + ".attn", heads, None, False, rope_base), True)
    x = _ln(x, sd, "encoder.norm")[:, 1 + nreg_enc:]
    # decoder tokens: register tokens at position (0, 0), patches at (row + 1, column + 1)
    nreg = sd["register_token"].shape[1]
    x = torch.cat((sd["register_token"].expand(b * f, -1, -1), x), dim=1)
    t = x.shape[1]
    yy, xx = torch.meshgrid(torch.arange(gh), torch.arange(gw), indexing="ij")
    if tile:
        assert nreg == 0 and gh % tile == 0 and gw % tile == 0
        pos = torch.stack((yy, xx), dim=-1).reshape(-1, 2)
    else:
        pos = torch.cat((torch.zeros((nreg, 2), dtype=torch.long), torch.stack((yy, xx), dim=-1).reshape(-1, 2) + 1), dim=0)
    pos = pos[None].expand(b * f, -1, -1).contiguous()
    pos_rows = pos                                    # what the head decoders see
    if tile:                                          # decoder: a frame's tokens and positions gathered into tile-major order
        perm = tile_major_index(gh, gw, tile)
        x, pos = x[:, perm], pos[:, perm]
    local_out = None
    for i in range(_count(sd, "local_decoder.")):
        pre = f"local_decoder.{i}"
        x = _block(x, sd, pre, lambda y: _dense_attention(y, sd, pre + ".attn", heads, pos, True, rope_base), True)
        local_out = x
        pre = f"global_decoder.{i}"
        a = pre + ".attn"

        def global_attention(y):
            out = sparse_layer(y.reshape(b, f * t, dim), sd[a + ".qkv.weight"], sd[a + ".qkv.bias"], sd[a + ".gate.0.weight"],
                               sd[a + ".gate.0.bias"], sd[a + ".proj.weight"], sd[a + ".proj.bias"], heads, block_tokens, topk,
                               xpos=pos.reshape(b, f * t, 2), qn_w=sd[a + ".q_norm.weight"], qn_b=sd[a + ".q_norm.bias"],
                               kn_w=sd[a + ".k_norm.weight"], kn_b=sd[a + ".k_norm.bias"], rope_base=rope_base, ln_eps=LN_EPS)
            return out["out"].reshape(b * f, t, dim)

        x = _block(x, sd, pre, global_attention, True)
    feat = torch.cat((local_out, x), dim=-1)
    if tile:                                          # back: the token at tile-major place i returns to row-major place perm[i]
        back = torch.empty_like(feat)
        back[:, perm] = feat
        feat, pos = back, pos_rows

    def head_decoder(name):
        y = F.linear(feat, sd[name + ".project.weight"], sd[name + ".project.bias"])
        for i in range(_count(sd, name + ".blocks.")):
            pre = f"{name}.blocks.{i}"
            y = _block(y, sd, pre, lambda z: _dense_attention(z, sd, pre + ".attn", heads, pos, False, rope_base), False)
        return F.linear(y, sd[name + ".linear_out.weight"], sd[name + ".linear_out.bias"])

    def pixel_head(tokens, name):
        y = F.linear(tokens, sd[name + ".proj.weight"], sd[name + ".proj.bias"]).transpose(-1, -2).reshape(b * f, -1, gh, gw)
        return F.pixel_shuffle(y, patch).permute(0, 2, 3, 1)

    pts = pixel_head(head_decoder("point_decoder")[:, nreg:], "point_head")
    conf = pixel_head(head_decoder("conf_decoder")[:, nreg:], "conf_head")
    cam = head_decoder("camera_decoder").mean(dim=1)
    p9 = F.linear(F.gelu(F.linear(cam, sd["camera_head.mlp.0.weight"], sd["camera_head.mlp.0.bias"])),
                  sd["camera_head.mlp.2.weight"], sd["camera_head.mlp.2.bias"])
    # rotation from two 3-vectors (offset towards the identity) by Gram-Schmidt, third axis by the cross product
    e1 = F.normalize(p9[:, 0:3] + torch.tensor([1.0, 0.0, 0.0]), dim=-1)
    v2 = p9[:, 3:6] + torch.tensor([0.0, 1.0, 0.0])
    e2 = F.normalize(v2 - (e1 * v2).sum(-1, keepdim=True) * e1, dim=-1)
    e3 = torch.linalg.cross(e1, e2)
    poses = torch.eye(4).repeat(b * f, 1, 1)
    poses[:, :3, :3] = torch.stack((e1, e2, e3), dim=-1)
    poses[:, :3, 3] = p9[:, 6:9]
    poses = poses.reshape(b, f, 4, 4)
    z = torch.exp(pts[..., 2:3])
    local_points = torch.cat((pts[..., :2] * z, z), dim=-1).reshape(b, f, gh * patch, gw * patch, 3)
    homog = torch.cat((local_points, torch.ones_like(local_points[..., :1])), dim=-1)
    points = torch.einsum("bnij,bnhwj->bnhwi", poses, homog)[..., :3]
    out = dict(points=points, local_points=local_points, conf=conf.reshape(b, f, gh * patch, gw * patch, 1), camera_poses=poses)
    if return_features:
        out["features"] = feat
    return out
