"""``SparseFlashAttentionRope``: the reference's global sparse attention layer
(pi3/models/layers/sparse_attention.py:60-141) on the HIP kernels of this package.

Same constructor arguments, same parameter names (``qkv``, ``proj``, ``q_norm``, ``k_norm``, ``gate.0``) and the
same ``forward(x, attn_bias=None, xpos=None)``, so a reference checkpoint loads with ``load_state_dict``.
Differences, all on the host side of the operator boundary:

* q, k, v are handed to the kernels as strided views of the packed projection (no ``.contiguous()`` copies),
  pooling reads the packed projection directly, and the gated merge runs in the selection kernel's epilogue
  (or in its own kernel where that is not built), writing ``[B, N, C]`` for ``proj``;
* when a gradient is wanted (grad mode on and the input or a parameter requires grad) the layer runs as a
  differentiable composition instead: the two attention operators with their backward kernels (bf16/fp16,
  head_dim 64, blocks of 64 or 16 tokens), pooling, norm/RoPE and merge as torch expressions;
* ``N`` need not be a multiple of the block: the last block pools its valid tokens, its keys beyond ``N`` are
  masked and its query rows beyond ``N`` do not exist (the reference raises for such ``N``);
* the top-k count, 32 in the reference, is a constructor argument.
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import Tensor, nn

from ..sparse_attn import ops
from ..sparse_attn.flash_attention_topk import flash_attn_topk_func
from .pos_embed import RoPE2D, block_positions


def norm_rope_fused_or_eager(t: Tensor, norm: nn.Module, rope, pos: Optional[Tensor], n_pos: Optional[int] = None) -> Tensor:
    """qk-norm, cast and RoPE of one ``[B,H,N,D]`` tensor (reference sparse_attention.py:103-110,120-124): one fused
    kernel where it is built -- a tensor on the GPU, head_dim 64, ``nn.Identity`` or an affine ``nn.LayerNorm`` of
    exactly that type, the package's RoPE2D or no rotation -- and the separate torch modules otherwise (any other norm
    module, a LayerNorm without affine parameters, another rope).  Same rounding points either way, except that the
    kernel takes the LayerNorm parameters in the tokens' dtype (fp32 parameters under autocast are rounded to it).
    ``n_pos``: number of rows of the kernel's cos/sin tables for THIS call (every coordinate in ``pos`` must be below it;
    the kernel clamps larger ones); default: the rope module's ``max_positions``, else ``pos.max() + 1`` (a device
    synchronisation)."""
    fused_norm = isinstance(norm, nn.Identity) or (type(norm) is nn.LayerNorm and norm.elementwise_affine)
    fused_rope = pos is None or isinstance(rope, RoPE2D)
    if t.is_cuda and t.shape[-1] == 64 and fused_norm and fused_rope and not (isinstance(norm, nn.Identity) and pos is None):
        cos = sin = None
        if pos is not None:
            rows = n_pos or rope.max_positions or int(pos.max()) + 1
            cos, sin = rope.tables(64, rows, t.device, t.dtype)
        ln = norm if isinstance(norm, nn.LayerNorm) else None
        out = ops.norm_rope(t, pos, cos, sin, ln.weight if ln is not None else None,
                            ln.bias if ln is not None else None, ln.eps if ln is not None else 0.0)
        if out is not None:
            return out
    t = norm(t).to(t.dtype)
    return rope(t, pos) if pos is not None else t


class SparseFlashAttentionRope(nn.Module):
    def __init__(
        self,
        dim: int,
        num_heads: int = 16,
        qkv_bias: bool = False,
        proj_bias: bool = True,
        attn_drop: float = 0.0,
        proj_drop: float = 0.0,
        qk_norm: bool = False,
        norm_layer=nn.LayerNorm,
        rope=None,
        block_size: int = 4,
        topk: int = 32,
    ) -> None:
        super().__init__()
        assert dim % num_heads == 0, "dim must be a multiple of num_heads"
        self.num_heads = num_heads
        head_dim = dim // num_heads
        self.scale = head_dim ** -0.5  # kept for parity with the reference; both operators default to it

        self.qkv = nn.Linear(dim, dim * 3, bias=qkv_bias)
        self.attn_drop = nn.Dropout(attn_drop)
        self.proj = nn.Linear(dim, dim, bias=proj_bias)
        self.proj_drop = nn.Dropout(proj_drop)
        self.q_norm = norm_layer(head_dim) if qk_norm else nn.Identity()
        self.k_norm = norm_layer(head_dim) if qk_norm else nn.Identity()
        self.rope = rope

        # gate: sigmoid(linear), weight 0 and bias (-1, +1) per head at initialisation
        gate_linear = nn.Linear(dim, num_heads * 2, bias=True)
        nn.init.zeros_(gate_linear.weight)
        with torch.no_grad():
            gate_linear.bias.copy_(torch.tensor([-1.0, 1.0]).repeat(num_heads))
        self.gate = nn.Sequential(gate_linear, nn.Sigmoid())
        self.block_size = block_size
        self.topk = topk
        self.keep_topk_idx = False   # debugging aid: keep the last forward's block indices in ``last_topk_idx``
        self.last_topk_idx = None
        self.last_prepass = None     # whether the last forward used the one-pass kernel over the packed projection
        self.last_path = None        # which route the last forward took: "fused-merge", "two-operators" or "autograd"

    def _norm_rope(self, t: Tensor, norm: nn.Module, pos: Optional[Tensor], n_pos: Optional[int] = None) -> Tensor:
        return norm_rope_fused_or_eager(t, norm, self.rope, pos, n_pos)

    def _prepass(self, qkv: Tensor, h: int, block: int, pos: Optional[Tensor], n_pos: Optional[int] = None):
        """The fused pre-pass where its conditions hold (those of ``norm_rope_fused_or_eager`` for both norms), else None."""
        def plain(norm):
            return isinstance(norm, nn.Identity) or (type(norm) is nn.LayerNorm and norm.elementwise_affine)
        same_kind = isinstance(self.q_norm, nn.Identity) == isinstance(self.k_norm, nn.Identity)
        if not (qkv.is_cuda and plain(self.q_norm) and plain(self.k_norm) and same_kind and (pos is None or isinstance(self.rope, RoPE2D))):
            return None
        if isinstance(self.q_norm, nn.Identity) and pos is None:   # nothing to do to q and k: the kernels read the projection in place
            return None
        if block < 32:   # many pooled tokens: the index kernel is long and starts earlier behind the separate pooling kernel,
            return None  # beside the norm/RoPE kernels (measured at 266 496 tokens, block 16: 10.9 against 11.2 ms per layer)
        cos = sin = None
        if pos is not None:
            rows = n_pos or self.rope.max_positions or int(pos.max()) + 1
            cos, sin = self.rope.tables(64, rows, qkv.device, qkv.dtype)
        ln = isinstance(self.q_norm, nn.LayerNorm)
        if ln and self.q_norm.eps != self.k_norm.eps:
            return None
        return ops.qkv_prepass(qkv, h, block, pos, cos, sin,
                               (self.q_norm.weight, self.q_norm.bias) if ln else None,
                               (self.k_norm.weight, self.k_norm.bias) if ln else None, self.q_norm.eps if ln else 0.0)

    def _forward_with_grad(self, x: Tensor, xpos: Optional[Tensor]) -> Tensor:
        """The same layer as a differentiable composition (training): the two attention operators carry their own
        backward kernels; pooling, qk-norm/RoPE and the gated merge run as the torch expressions of the reference
        (sparse_attention.py:97-110,120-136), whose gradients autograd provides."""
        b, n, c = x.shape
        h = self.num_heads
        d = c // h
        block = self.block_size ** 2
        nc = -(-n // block)
        qkv = self.qkv(x)
        gate = self.gate(x).view(b, n, h, 2).permute(0, 2, 1, 3)              # [B, H, N, 2]
        q, k, v = qkv.view(b, n, 3, h, d).permute(2, 0, 3, 1, 4).unbind(0)    # each [B, H, N, D]

        def pool(t):  # block means; a ragged tail block averages its valid tokens
            pad = nc * block - n
            tf = torch.nn.functional.pad(t, (0, 0, 0, pad)) if pad else t
            sums = tf.reshape(b, h, nc, block, d).float().sum(dim=3)
            counts = torch.full((nc, 1), float(block), device=t.device)
            if pad:
                counts[-1] = float(block - pad)
            return (sums / counts).to(t.dtype)

        def norm_rope(t, norm, pos):
            t = norm(t).to(t.dtype)
            return self.rope(t, pos) if pos is not None else t

        use_pos = xpos is not None and self.rope is not None
        pos_c = block_positions(xpos, block) if use_pos else None
        q_c, k_c, v_c = pool(q), pool(k), pool(v)
        q_c, k_c = norm_rope(q_c, self.q_norm, pos_c), norm_rope(k_c, self.k_norm, pos_c)
        o_c, idx = flash_attn_topk_func(q_c, k_c, v_c, self.topk)
        if self.keep_topk_idx:
            self.last_topk_idx = idx
        pos = xpos if use_pos else None
        q, k = norm_rope(q, self.q_norm, pos), norm_rope(k, self.k_norm, pos)
        o_s = ops.select_attn_autograd(q, k, v, idx, block)
        blk = torch.arange(n, device=x.device) // block
        out = gate[..., 0:1] * o_c[:, :, blk] + gate[..., 1:2] * o_s           # [B, H, N, D]
        out = out.permute(0, 2, 1, 3).reshape(b, n, c)
        return self.proj_drop(self.proj(out))

    def forward(self, x: Tensor, attn_bias=None, xpos: Optional[Tensor] = None, n_pos: Optional[int] = None) -> Tensor:
        """``n_pos`` (optional, beyond the reference's signature): an upper bound, exclusive, of the coordinates in
        ``xpos`` for this call; sizes the fused kernels' cos/sin tables without a device synchronisation and without
        touching state shared between calls."""
        if torch.is_grad_enabled() and (x.requires_grad or any(p.requires_grad for p in self.parameters())):
            self.last_path = "autograd"
            return self._forward_with_grad(x, xpos)
        b, n, c = x.shape
        h = self.num_heads
        d = c // h
        block = self.block_size ** 2

        qkv = self.qkv(x)                                              # [B, N, 3C], layout (qkv h d)
        gate = self.gate(x).view(b, n, h, 2).permute(0, 2, 1, 3)       # [B, H, N, 2], strided view

        use_pos = xpos is not None and self.rope is not None
        pos = xpos if use_pos else None
        # One pass over the packed projection: block means of the raw q, k, v (compressed branch) and norm + RoPE of
        # the full-token q and k (selection branch), each input row read once.  Where that kernel is not built
        # (head_dim other than 64, another norm or rope module): pooling kernel, then norm/RoPE per tensor.
        pre = self._prepass(qkv, h, block, pos, n_pos)
        self.last_prepass = pre is not None
        if pre is not None:
            q, k, v, q_c, k_c, v_c = pre
        else:
            q_c, k_c, v_c = ops.pool_qkv_packed(qkv, h, block)
        # compressed branch: pooled raw projections -> norm -> RoPE at block positions -> attention + top-k
        pos_c = block_positions(xpos, block) if use_pos else None
        q_c, k_c = self._norm_rope(q_c, self.q_norm, pos_c, n_pos), self._norm_rope(k_c, self.k_norm, pos_c, n_pos)
        # the index kernel needs pooled q and k only and its result is first read by the selection kernel: where
        # it is a kernel of its own it runs on a second stream, beside the compressed attention (and the norm/RoPE of
        # the full tokens where they are separate kernels)
        side = x.is_cuda and ops._two_kernel_compressed(q_c, self.topk)
        if side:
            idx, join = ops.topk_indices_on_side_stream(q_c, k_c, self.topk)
            o_c, _ = ops.compressed_attn_topk(q_c, k_c, v_c, None)
        else:
            o_c, idx = flash_attn_topk_func(q_c, k_c, v_c, self.topk)

        if pre is None:  # selection branch on strided views of the projection; norm/RoPE make q, k contiguous
            q, k, v = qkv.view(b, n, 3, h, d).permute(2, 0, 3, 1, 4).unbind(0)   # each [B, H, N, D]
            q, k = self._norm_rope(q, self.q_norm, pos, n_pos), self._norm_rope(k, self.k_norm, pos, n_pos)
        if side:
            join()
        if self.keep_topk_idx:
            self.last_topk_idx = idx

        out = ops.select_attn_merge(q, k, v, idx, o_c, gate, block)
        self.last_path = "fused-merge"
        if out is None:
            self.last_path = "two-operators"
            out = ops.gated_merge(o_c, ops.select_attn(q, k, v, idx, block), gate, block)

        out = self.proj(out)
        return self.proj_drop(out)
