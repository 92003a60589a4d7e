#!/usr/bin/env python3
"""Benchmark of the sparse global-attention layer path on one MI355X.

A step is one pass of the hot path (pool q,k,v -> compressed attention + top-k -> selection
attention -> gated merge) over one synthetic layer input already resident in HBM.  The default
workload is the headline configuration: 256 frames x 1041 tokens = 266 496 tokens, 16 heads x 64,
block 64, top-k 16, bf16, seeded low-rank-plus-noise q/k/v.

Prints ONE JSON line: ms/layer as `value`, effective TFLOP/s, per-kernel times measured with HIP
events on the launch stream, the roofline of the dominant (selection) kernel from its algorithmic
FLOPs, and a CPU baseline (the Python oracle timed on this host's cores on a bounded sample).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0
# (config, top-k, block, merge fused) -> HBM bytes per launch of the selection kernel and the profile summary they come from
MEASURED_TRAFFIC = {
    ("cfg3", 16, 64, True): (2.34e9, "profiles/select_merge_cfg3_256f_bf16_hbm_bytes.md"),
    ("cfg4", 16, 64, True): (9.48e9, "profiles/layer_cfg4_1000f_bf16_kernel_stats.md"),
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # The chip's clock governor needs some tens of back-to-back launches to settle under this load (the first
    # launches after an idle period run up to 40 % slower), so the default warm-up is long; a step is 1.8 ms.
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--config", default="cfg3", choices=["cfg1", "cfg2", "cfg3", "cfg4", "cfg5"],
                    help="cfg1-cfg4: one sparse global-attention layer call; cfg5: end-to-end Pi3_Sparse-style forward (frames/s)")
    ap.add_argument("--frames", type=int, default=100, help="cfg5: number of 518x392 frames")
    ap.add_argument("--topk", type=int, default=None)
    ap.add_argument("--block", type=int, default=64, choices=[16, 64],
                    help="tokens per block: 64 (the headline workload) or 16 (the reference layer's own block size, with --topk 32)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-heads", type=int, default=16, help="heads of the workload the CPU baseline runs")
    ap.add_argument("--materialize-scores", action="store_true", help="force the two-kernel score/top-k path")
    ap.add_argument("--no-fuse-merge", action="store_true", help="run selection attention and the gated merge as two kernels")
    ap.add_argument("--no-overlap", action="store_true",
                    help="run every kernel on one stream (per-kernel times for pooling and the compressed branch); by default "
                         "the index kernel runs on a second stream beside the pooling of v and the compressed attention")
    ap.add_argument("--backward", action="store_true",
                    help="time the backward of the two attention operators (one JSON line of its own; not the headline metric)")
    ap.add_argument("--only", default=None, choices=["pool", "compressed_topk", "select", "merge", "select_merge", "prepass", "copy"],
                    help="profiling aid: after one full pass, launch only this stage `steps` times (no JSON line)")
    return ap.parse_args()


def _cpu_model() -> str:
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(q, k, v, gate, block, topk, heads):
    """Times the oracle (eager fp32 PyTorch + numpy top-k) on `heads` heads of the workload, on as many threads as
    this process may use (its CPU affinity, not the machine's core count: the box's share can be smaller)."""
    import torch

    import oracle

    usable = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    threads = max(1, min(usable, int(os.environ.get("OMP_NUM_THREADS", usable))))
    torch.set_num_threads(threads)
    hs = slice(0, heads)
    qs, ks, vs, gs = (t[:, hs].float() for t in (q, k, v, gate))
    t0 = time.perf_counter()
    oracle.sparse_global_attention(qs, ks, vs, gs, block, topk)
    dt = time.perf_counter() - t0
    total_heads = q.shape[1]
    return {
        "value": dt * 1e3 * total_heads / heads,
        "unit": "ms",
        "cores": torch.get_num_threads(),
        "host_cpus": os.cpu_count(),
        "cpu_model": _cpu_model(),
        "kind": "port",
        "sample": f"oracle (eager fp32 PyTorch + numpy top-k) on heads 0..{heads - 1} of {total_heads}, all tokens: "
                  f"{dt:.2f} s measured, scaled x{total_heads // heads} to the full layer",
    }


def _prepass_stage(qd, kd, vd, block):
    """The layer's one-pass kernel over a packed [1, N, 3*H*64] projection built from the workload's q, k, v: block
    means of the raw rows + LayerNorm + RoPE2D of q and k (positions of a 37 x 28 patch grid after 5 register tokens)."""
    import torch

    from speed3r_amd.layers import RoPE2D
    from speed3r_amd.sparse_attn import ops

    _, h, n, d = qd.shape
    packed = torch.stack((qd[0], kd[0], vd[0]), dim=0).permute(2, 0, 1, 3).reshape(1, n, 3 * h * d).contiguous()
    t = torch.arange(n, device=qd.device) % 1041
    patch = (t - 5).clamp(min=0)
    pos = torch.where((t >= 5)[:, None], torch.stack((patch // 28 + 1, patch % 28 + 1), dim=-1), torch.zeros_like(t)[:, None])[None]
    cos, sin = RoPE2D(100.0).tables(64, 39, qd.device, qd.dtype)
    g = torch.Generator().manual_seed(9)
    ln = [((1 + 0.1 * torch.randn(64, generator=g)).to(qd.dtype).to(qd.device), (0.1 * torch.randn(64, generator=g)).to(qd.dtype).to(qd.device))
          for _ in range(2)]
    return lambda: ops.qkv_prepass(packed, h, block, pos, cos, sin, ln[0], ln[1], 1e-6)


def run_end_to_end(args) -> int:
    """cfg5: random-init Pi3_Sparse-style model, bf16, synthetic frames in [0,1]; frames/s and the share of GPU time
    spent in the sparse global attention (HIP events around the 18 global attention modules)."""
    import torch

    from speed3r_amd.model import Pi3SparseLike

    dev = torch.device("cuda:0")
    torch.manual_seed(4)
    model = Pi3SparseLike().to(torch.bfloat16).to(dev).eval()
    g = torch.Generator().manual_seed(4)
    imgs = torch.rand((1, args.frames, 3, 518, 392), generator=g).to(dev)
    spans = []

    def pre(_m, _a, _k=None):
        e = torch.cuda.Event(enable_timing=True)
        e.record()
        spans.append([e, None])

    def post(_m, _a, _o):
        e = torch.cuda.Event(enable_timing=True)
        e.record()
        spans[-1][1] = e

    for blk in model.global_decoder:
        blk.attn.register_forward_pre_hook(pre)
        blk.attn.register_forward_hook(post)
    steps, warmup = min(args.steps, 5), min(args.warmup, 2)
    with torch.no_grad():
        for _ in range(max(warmup, 1)):
            model(imgs)
        torch.cuda.synchronize()
        spans.clear()
        t0 = time.perf_counter()
        for _ in range(steps):
            out = model(imgs)
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
    sparse_ms = sum(a.elapsed_time(b) for a, b in spans) / steps
    ms = wall * 1e3 / steps
    tokens = args.frames * 1041
    print(json.dumps({
        "metric": "frames/s, Pi3_Sparse-style forward (ViT-L/14 encoder + 36-layer decoder + heads), bf16",
        "value": args.frames / (ms * 1e-3), "unit": "frames/s", "n_gpus": 1, "steps": steps, "warmup": max(warmup, 1),
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"cfg5: {args.frames} frames 518x392 -> {tokens} tokens (5 register + 1036 patch per frame), "
                               "18 frame-local dense + 18 global sparse attention layers (block 64, top-k 16), random-init weights",
                   "tokens": tokens, "block": 64, "topk": 16},
        "sparse_attention_ms": sparse_ms, "sparse_attention_share": sparse_ms / ms,
        "sparse_attention_ms_per_layer": sparse_ms / len(model.global_decoder),
        "peak_mem_gb": torch.cuda.max_memory_allocated() / 1e9,
        "outputs": {k: list(v.shape) for k, v in out.items()},
    }))
    return 0


def run_backward(args, cfg, qd, kd, vd, block, topk) -> int:
    """Backward of the selection operator and of the compressed (dense) operator on the forward's tensors: HIP events
    around delta, the key-centric lists (`s3r_key_block_lists`), the dQ kernel and the dK/dV kernel."""
    import torch

    import speed3r_amd as s3r
    from speed3r_amd import workloads
    from speed3r_amd.sparse_attn import ops

    n = cfg.tokens
    nkb = -(-n // block)
    with torch.no_grad():
        qc, kc, vc = s3r.pool_mean(qd, block), s3r.pool_mean(kd, block), s3r.pool_mean(vd, block)
        oc, idx, lsec = s3r.compressed_attn_topk(qc, kc, vc, topk, return_lse=True)
        o, lse = s3r.select_attn(qd, kd, vd, idx, block, return_lse=True)
        g = torch.randn(o.shape, generator=torch.Generator().manual_seed(7)).to(o.dtype).to(o.device)
        gc = torch.randn(oc.shape, generator=torch.Generator().manual_seed(8)).to(oc.dtype).to(oc.device)
        names = ["delta", "key_lists", "dq", "dkdv", "compressed_bwd"]

        def step(ev=None):
            def mark(i):
                if ev is not None:
                    ev[i].record()
            mark(0)
            delta = ops.attn_bwd_delta(o, g)
            mark(1)
            lists = ops.key_block_lists(idx, nkb)
            mark(2)
            dq, _, _ = ops.attn_bwd(qd, kd, vd, o, g, lse, idx, block, need_dkv=False, delta=delta)
            mark(3)
            _, dk, dv = ops.attn_bwd(qd, kd, vd, o, g, lse, idx, block, need_dq=False, delta=delta, key_lists=lists)
            mark(4)
            ops.attn_bwd(qc, kc, vc, oc, gc, lsec)
            mark(5)

        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        evs = [[torch.cuda.Event(enable_timing=True) for _ in range(6)] for _ in range(args.steps)]
        t0 = time.perf_counter()
        for i in range(args.steps):
            step(evs[i])
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
    ms = wall * 1e3 / args.steps
    kern = {nm: sum(e[i].elapsed_time(e[i + 1]) for e in evs) / args.steps for i, nm in enumerate(names)}
    mm = workloads.selection_flops(n, topk, block=block) / 2          # one product over the selected (query block, key block) pairs
    f_dq, f_dkdv = 3 * mm, 4 * mm
    dom = "dkdv" if kern["dkdv"] >= kern["dq"] else "dq"
    tfl = (f_dkdv if dom == "dkdv" else f_dq) / (kern[dom] * 1e-3) / 1e12
    print(json.dumps({
        "metric": "ms/layer backward (selection + compressed attention operators), global sparse attn @%d frames bf16" % cfg.frames,
        "value": ms, "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{cfg.name} backward: {n} tokens, 16 heads x 64, block {block}, top-k {topk}, B=1"},
        "kernels_ms": kern,
        "effective_tflops": (f_dq + f_dkdv + 2.5 * workloads.compressed_flops(n, block=block)) / (ms * 1e-3) / 1e12,
        "roofline": {"kernel": "bwd_dkdv_kernel" if dom == "dkdv" else "bwd_dq_kernel", "bound": "mfma", "achieved": tfl,
                     "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": tfl / PEAK_BF16_TFLOPS, "traffic": None},
    }))
    return 0


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on one GPU only (got --gpus {args.gpus}); the path shards by head "
              "without collectives (heads are independent in every kernel)", file=sys.stderr)
        return 2

    import torch

    import speed3r_amd as s3r
    from speed3r_amd import workloads

    assert torch.cuda.is_available(), "bench.py needs a HIP device"
    if args.config == "cfg5":
        return run_end_to_end(args)
    dev = torch.device("cuda:0")
    cfg, q, k, v, gate = workloads.make_config(args.config)
    topk = args.topk or cfg.topk
    block = args.block
    n = cfg.tokens
    qd, kd, vd, gd = (t.to(dev) for t in (q, k, v, gate))
    mat = True if args.materialize_scores else None

    fused = not args.no_fuse_merge
    overlap = not args.no_overlap and not args.materialize_scores and cfg.dtype != torch.float32 and topk in (1, 2, 4, 8, 16, 32)

    def step(timeline=None):
        return s3r.sparse_global_attention(qd, kd, vd, gd, block, topk, materialize_scores=mat, fuse_merge=fused,
                                           overlap=overlap, timeline=timeline)

    if args.backward:
        return run_backward(args, cfg, qd, kd, vd, block, topk)

    if args.only:
        with torch.no_grad():
            qc, kc, vc = s3r.pool_mean(qd, block), s3r.pool_mean(kd, block), s3r.pool_mean(vd, block)
            o_cmp, idx = s3r.compressed_attn_topk(qc, kc, vc, topk, materialize_scores=mat)
            o_sel = s3r.select_attn(qd, kd, vd, idx, block)
            stage = {
                "pool": lambda: s3r.pool_mean(qd, block),
                "compressed_topk": lambda: s3r.compressed_attn_topk(qc, kc, vc, topk, materialize_scores=mat),
                "select": lambda: s3r.select_attn(qd, kd, vd, idx, block),
                "merge": lambda: s3r.gated_merge(o_cmp, o_sel, gd, block),
                "select_merge": lambda: s3r.select_attn_merge(qd, kd, vd, idx, o_cmp, gd, block),
                # a plain device copy of q (reads and writes q.nbytes): the yardstick for the HBM byte counters
                "copy": lambda: torch.empty_like(qd).copy_(qd),
                "prepass": _prepass_stage(qd, kd, vd, block),
            }[args.only]
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                stage()
            torch.cuda.synchronize()
            print(f"{args.only}: {(time.perf_counter() - t0) * 1e3 / args.steps:.4f} ms per launch", file=sys.stderr)
        return 0

    with torch.no_grad():
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        evs = [{} for _ in range(args.steps)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            step(evs[i])
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        peak_mem = torch.cuda.max_memory_allocated()

    ms_per_step = wall * 1e3 / args.steps
    nc = -(-n // block)
    def span(a, b):
        return sum(e[a].elapsed_time(e[b]) for e in evs) / args.steps

    fused = fused and "merge" not in evs[0]   # the merge runs in the selection kernel's epilogue only where that is built
    sel_name = "select_merge" if fused else "select"
    if overlap:   # the index kernel runs on a second stream beside the pooling of v and the compressed attention
        kern_ms = {"pool+compressed_topk (two streams)": span("start", "select")}
    else:
        kern_ms = {"pool": span("start", "pooled"), "compressed_topk": span("pooled", "select")}
    if fused:
        kern_ms["select_merge"] = span("select", "end")
    else:
        kern_ms["select"] = span("select", "merge")
        kern_ms["merge"] = span("merge", "end")
    f_sel = workloads.selection_flops(n, topk, block=block)
    f_cmp = workloads.compressed_flops(n, block=block)
    sel_tflops = f_sel / (kern_ms[sel_name] * 1e-3) / 1e12
    es = 2 if cfg.dtype != torch.float32 else 4
    pool_bytes = 3 * (n + nc) * 16 * 64 * es
    merge_bytes = (2 * n * 16 * 64 + n * 16 * 2 + nc * 16 * 64) * es

    result = {
        "metric": "ms/layer, global sparse attn @%d frames %s" % (cfg.frames, "bf16" if es == 2 else "fp32"),
        "value": ms_per_step,
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if es == 2 else "f32",
        "data": "synthetic",
        "config": {
            "workload": f"{cfg.name}: {cfg.frames} frames x {workloads.TOKENS_PER_FRAME} tokens = {n} tokens, "
                        f"16 heads x 64, block {block}, top-k {topk}, B=1",
            "tokens": n, "heads": 16, "head_dim": 64, "block": block, "topk": topk,
            "scores": "materialized" if args.materialize_scores else "fused (never leave the chip)",
        },
        "effective_tflops": (f_sel + f_cmp) / (ms_per_step * 1e-3) / 1e12,
        "kernels_ms": kern_ms,
        "hbm_gbs": {**({} if overlap else {"pool": pool_bytes / (kern_ms["pool"] * 1e-3) / 1e9}),
                    **({} if fused else {"merge": merge_bytes / (kern_ms["merge"] * 1e-3) / 1e9})},
        "peak_mem_gb": peak_mem / 1e9,
        "roofline": {
            "kernel": ("select_pipe_kernel" if block == 64 else "select_b16_kernel") + (" (gated merge in its epilogue)" if fused else ""),
            "bound": "mfma",
            "achieved": sel_tflops,
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": sel_tflops / PEAK_BF16_TFLOPS,
            # HBM bytes per launch: not measured inside this run; the figure is the one rocprofv3 FETCH_SIZE / WRITE_SIZE
            # gave for this kernel on this workload, scaled by a plain copy (file named in traffic_source)
            "traffic": MEASURED_TRAFFIC.get((args.config, topk, block, fused), (None, None))[0],
            "traffic_source": MEASURED_TRAFFIC.get((args.config, topk, block, fused), (None, None))[1],
        },
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(q, k, v, gate, block, topk, args.cpu_heads)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
