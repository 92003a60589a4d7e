"""Writes tests/golden/sparse_path_small.npz: stage-by-stage vectors for the sparse attention path.

The reference ships no golden vectors for this path and its kernels cannot run without a
GPU, so these vectors come from brute force written here, independently of ``oracle/`` and of
the HIP kernels: fp64 means, fp64 dense softmax attention (stored rounded to fp32) under an explicit multiplicity
mask, and a pure-Python sort on (sortable key, column) for the top-k.  Inputs are stored as
bf16 bit patterns (uint16) so every consumer sees identical values.

Run from the repository root:  python tests/golden/make_fixtures.py
"""
from __future__ import annotations

import struct
from pathlib import Path

import numpy as np
import torch

OUT = Path(__file__).resolve().parent / "sparse_path_small.npz"

H, N, D, BS, K = 2, 200, 64, 64, 2   # 3 full blocks + a ragged tail of 8 tokens


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16).copy()


def py_sort_key(x: float) -> int:
    bits = struct.unpack("<I", struct.pack("<f", x))[0]
    return (~bits & 0xFFFFFFFF) if bits >> 31 else (bits | 0x80000000)


def brute_topk(scores: np.ndarray, k: int) -> np.ndarray:
    rows, cols = scores.shape
    out = np.empty((rows, k), dtype=np.int32)
    for r in range(rows):
        order = sorted(range(cols), key=lambda j: (-py_sort_key(float(scores[r, j])), j))
        order = (order + [cols - 1] * k)[:k]      # fewer columns than k: filler is the last column
        out[r] = order
    return out


def main() -> None:
    g = torch.Generator().manual_seed(20240607)
    q = (torch.randn((1, H, N, D), generator=g) / 4).to(torch.bfloat16)
    k = (torch.randn((1, H, N, D), generator=g) / 4).to(torch.bfloat16)
    v = torch.randn((1, H, N, D), generator=g).to(torch.bfloat16)
    gate = torch.sigmoid(torch.randn((1, H, N, 2), generator=g)).to(torch.bfloat16)
    nc = -(-N // BS)
    scale = 1.0 / D ** 0.5

    # stage 1: pooling, fp64 means over valid tokens
    def pool64(x):
        x = x.to(torch.float64)
        return torch.stack([x[:, :, j * BS:min(N, (j + 1) * BS)].mean(dim=2) for j in range(nc)], dim=2)
    pooled = {name: pool64(t) for name, t in (("q", q), ("k", k), ("v", v))}

    # stage 2: compressed attention on a separate, larger pooled-shaped input (Lq=Lk=150: 2 full tiles + tail)
    lc = 150
    qc = (torch.randn((1, H, lc, D), generator=g) / 2).to(torch.bfloat16)
    kc = (torch.randn((1, H, lc, D), generator=g) / 2).to(torch.bfloat16)
    vc = torch.randn((1, H, lc, D), generator=g).to(torch.bfloat16)
    s64 = qc.to(torch.float64) @ kc.to(torch.float64).transpose(-1, -2)
    p64 = torch.softmax(s64 * scale, dim=-1)
    oc64 = p64 @ vc.to(torch.float64)
    lse64 = torch.logsumexp(s64 * scale, dim=-1)

    # stage 3: top-k on explicit fp32 scores: smooth random rows, tie-heavy integer rows, signed zeros
    rng = np.random.default_rng(7)
    smooth = rng.standard_normal((24, 300)).astype(np.float32)
    ties = rng.integers(-3, 4, size=(24, 300)).astype(np.float32)
    zeros = np.zeros((4, 70), dtype=np.float32)
    zeros[:, ::3] = -0.0
    zeros[1, 5] = 1.0
    zeros[2, :] = -0.0
    zeros[2, 69] = 0.0
    short = rng.standard_normal((4, 5)).astype(np.float32)   # fewer columns than k
    topk_cases = {"smooth": (smooth, 16), "ties": (ties, 16), "zeros": (zeros, 8), "short": (short, 8)}

    # stage 4: selection with explicit indices incl. a duplicate, a skip (-1) and the ragged block
    idx = torch.tensor([[[[0, 1], [1, 1], [3, 0], [-1, 2]],
                         [[2, 3], [0, -1], [1, 2], [3, 3]]]], dtype=torch.int32)
    o_sel64 = torch.zeros((1, H, N, D), dtype=torch.float64)
    for h in range(H):
        s = (q[0, h].to(torch.float64) @ k[0, h].to(torch.float64).T) * scale
        mult = torch.zeros((N, N), dtype=torch.float64)
        for m in range(nc):
            for j in idx[0, h, m].tolist():
                if j < 0 or j * BS >= N:
                    continue
                mult[m * BS:min(N, (m + 1) * BS), j * BS:min(N, (j + 1) * BS)] += 1
        w = torch.exp(torch.where(mult > 0, s, torch.full_like(s, -1e300)) - s.max()) * mult
        o_sel64[0, h] = (w @ v[0, h].to(torch.float64)) / w.sum(dim=-1, keepdim=True)

    # stage 5: merge in bf16 with per-op rounding, written element by element
    o_cmp_b = oc64[:, :, :nc].to(torch.bfloat16)     # any bf16 tensor of pooled shape will do
    o_sel_b = o_sel64.to(torch.bfloat16)
    merged = torch.empty((1, N, H * D), dtype=torch.bfloat16)
    for h in range(H):
        for n in range(N):
            a = (gate[0, h, n, 0].float() * o_cmp_b[0, h, n // BS].float()).to(torch.bfloat16)
            c = (gate[0, h, n, 1].float() * o_sel_b[0, h, n].float()).to(torch.bfloat16)
            merged[0, n, h * D:(h + 1) * D] = (a.float() + c.float()).to(torch.bfloat16)

    arrays = dict(
        meta=np.array([H, N, D, BS, K, lc], dtype=np.int64),
        q=bf16_bits(q), k=bf16_bits(k), v=bf16_bits(v), gate=bf16_bits(gate),
        pooled_q=pooled["q"].numpy().astype(np.float32), pooled_k=pooled["k"].numpy().astype(np.float32),
        pooled_v=pooled["v"].numpy().astype(np.float32),
        qc=bf16_bits(qc), kc=bf16_bits(kc), vc=bf16_bits(vc),
        cmp_scores=s64.numpy().astype(np.float32), cmp_out=oc64.numpy().astype(np.float32),
        cmp_lse=lse64.numpy().astype(np.float32),
        sel_idx=idx.numpy(), sel_out=o_sel64.numpy().astype(np.float32),
        merge_o_cmp=bf16_bits(o_cmp_b), merge_o_sel=bf16_bits(o_sel_b), merge_out=bf16_bits(merged),
    )
    for name, (sc, kk) in topk_cases.items():
        arrays[f"topk_{name}_scores"] = sc
        arrays[f"topk_{name}_idx"] = brute_topk(sc, kk)
    np.savez_compressed(OUT, **arrays)
    print("wrote", OUT, OUT.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
