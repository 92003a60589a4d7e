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
@pytest.mark.parametrize("n,block_size,topk", [(320, 8, 2), (200, 8, 4), (160, 4, 4), (64, 8, 1)])
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


def test_layer_is_forward_only():
    m = _make(128, 2, 8, 2, torch.bfloat16, seed=7).to(DEV)
    x = torch.randn((1, 128, 128), device=DEV, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError):
        m(x)                      # parameters require grad and grad mode is on
