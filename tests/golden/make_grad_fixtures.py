"""Writes tests/golden/sparse_path_grads_small.npz: gradients of the selection attention for 16- and 64-token blocks.

The reference ships no golden vectors, and its backward kernels need Triton and a GPU, so these come from brute
force written here, independently of ``oracle/`` and of the HIP kernels: the forward is a dense fp64 softmax over
all keys under an explicit multiplicity matrix (how many times query i attends key j: duplicates count twice,
skipped entries not at all), differentiated by torch autograd in fp64; gradients are stored rounded to fp32.  Inputs
and the output gradient are stored as bf16 bit patterns (uint16) so every consumer sees identical values.

Run from the repository root:  python tests/golden/make_grad_fixtures.py
"""
from __future__ import annotations

from pathlib import Path

import numpy as np
import torch

OUT = Path(__file__).resolve().parent / "sparse_path_grads_small.npz"

H, N, D = 2, 104, 64   # 6 blocks of 16 and a ragged one of 8; one block of 64 and a ragged one of 40


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16).copy()


def grads(q, k, v, dout, idx, block):
    scale = 1.0 / D ** 0.5
    nb = -(-N // block)
    outs = []
    for h in range(H):
        mult = torch.zeros((N, N), dtype=torch.float64)
        for m in range(nb):
            for j in idx[0, h, m].tolist():
                if j < 0 or j * block >= N:
                    continue
                mult[m * block:min(N, (m + 1) * block), j * block:min(N, (j + 1) * block)] += 1
        qq, kk, vv = (t[0, h].to(torch.float64).requires_grad_(True) for t in (q, k, v))
        s = (qq @ kk.T) * scale
        w = torch.exp(s - s.detach().max()) * mult          # the shift cancels in the ratio below
        den = w.sum(dim=-1, keepdim=True)
        o = torch.where(den > 0, w @ vv / torch.where(den > 0, den, torch.ones_like(den)), torch.zeros_like(w @ vv))
        o.backward(dout[0, h].to(torch.float64))
        outs.append((o.detach(), qq.grad, kk.grad, vv.grad))
    return [torch.stack([x[i] for x in outs])[None].to(torch.float32).numpy() for i in range(4)]


def main() -> None:
    g = torch.Generator().manual_seed(20240611)
    q = (torch.randn((1, H, N, D), generator=g) / 2).to(torch.bfloat16)
    k = (torch.randn((1, H, N, D), generator=g) / 2).to(torch.bfloat16)
    v = torch.randn((1, H, N, D), generator=g).to(torch.bfloat16)
    dout = torch.randn((1, H, N, D), generator=g).to(torch.bfloat16)
    arrays = dict(meta=np.array([H, N, D], dtype=np.int64), q=bf16_bits(q), k=bf16_bits(k), v=bf16_bits(v), dout=bf16_bits(dout))
    # 16-token blocks: 7 query blocks x 3 entries with a skip, duplicates, the ragged block and an empty row
    idx16 = torch.randint(0, 7, (1, H, 7, 3), generator=g, dtype=torch.int32)
    idx16[0, 0, 1] = torch.tensor([6, 6, 2])
    idx16[0, 0, 3, 1] = -1
    idx16[0, 1, 2] = -1
    idx16[0, 1, 5] = torch.tensor([4, 9, 4])       # 9: beyond the sequence, skipped
    # 64-token blocks: 2 query blocks x 2 entries
    idx64 = torch.tensor([[[[0, 1], [1, 1]], [[1, -1], [0, 1]]]], dtype=torch.int32)
    for name, idx, block in (("b16", idx16, 16), ("b64", idx64, 64)):
        o, dq, dk, dv = grads(q, k, v, dout, idx, block)
        arrays.update({f"{name}_idx": idx.numpy(), f"{name}_out": o, f"{name}_dq": dq, f"{name}_dk": dk, f"{name}_dv": dv})
    np.savez_compressed(OUT, **arrays)
    print("wrote", OUT, OUT.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
