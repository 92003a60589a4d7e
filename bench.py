#!/usr/bin/env python3
"""Benchmark of the sparse global-attention layer path on one MI355X.

A step is one pass of the hot path (pool q,k,v -> compressed attention + top-k -> selection
attention -> gated merge) over one synthetic layer input already resident in HBM.  The default
workload is the headline configuration: 256 frames x 1041 tokens = 266 496 tokens, 16 heads x 64,
block 64, top-k 16, bf16, seeded low-rank-plus-noise q/k/v.

Prints ONE JSON line: ms/layer as `value`, effective TFLOP/s, per-kernel times measured with HIP
events on the launch stream (mean and median), the roofline of the dominant (selection) kernel from
its algorithmic FLOPs, and a CPU baseline (the Python oracle timed on this host's cores on a bounded
sample).  The default run appends, each from a short timed loop of its own after the headline region:
GB/s of the HBM-bound kernels on one stream (`hbm_gbs`), the 1000-frame layer (`cfg4`) and the
end-to-end model (`cfg5`: frames/s and the share of time inside the sparse attention modules).

The chip's clock governor needs some tens of back-to-back launches to settle under this load (the
first launches after an idle period run up to 40 % slower), so every timed loop is preceded by a
fixed number of untimed settling steps (`settle_steps` in the JSON) on top of `--warmup`.
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
SETTLE_STEPS = 40           # untimed steps in front of --warmup (clock governor), fixed
# (config, top-k, block, merge fused) -> HBM bytes per launch of the selection kernel, the profile summary they come from
# and the commit whose kernel was measured (the bytes are a property of the access pattern: list walk, tile size, merge
# in the epilogue; a change of those makes the figure stale)
MEASURED_TRAFFIC = {
    ("cfg3", 16, 64, True): (2.34e9, "profiles/select_merge_cfg3_256f_bf16_hbm_bytes.md (kernel of commit 771ade2)"),
    ("cfg4", 16, 64, True): (9.48e9, "profiles/layer_cfg4_1000f_bf16_kernel_stats.md (kernel of commit e9a5029: same list walk and tiles)"),
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-extras", action="store_true",
                    help="headline region only: no hbm_gbs / cfg4 / cfg5 loops after it (profiling runs)")
    ap.add_argument("--config", default="cfg3", choices=["cfg1", "cfg2", "cfg3", "cfg4", "cfg5"],
                    help="cfg1-cfg4: one sparse global-attention layer call; cfg5: end-to-end Pi3_Sparse-style forward (frames/s)")
    ap.add_argument("--frames", type=int, default=100, help="cfg5: number of 518x392 frames")
    ap.add_argument("--reference-setting", action="store_true",
                    help="cfg5 in the reference model's own setting: 504x392 frames (a multiple of 56), no register tokens, "
                         "4x4-tile-major token order, 16-token blocks, top-k 32")
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


def run_end_to_end(args, steps=None, warmup=None, reference_setting=None) -> dict:
    """cfg5: random-init Pi3_Sparse-style model, bf16, synthetic frames in [0,1]; frames/s and the share of GPU time
    spent in the sparse global attention (HIP events around the 18 global attention modules)."""
    import torch

    from speed3r_amd.model import Pi3SparseLike

    dev = torch.device("cuda:0")
    torch.manual_seed(4)
    ref = args.reference_setting if reference_setting is None else reference_setting
    hh, ww = (504, 392) if ref else (518, 392)
    if ref:   # pi3/models/pi3_sparse.py:29-71,163-169; pi3/models/layers/sparse_attention.py:73,98,112
        model = Pi3SparseLike(grid=(36, 28), num_register=0, token_order="tile", block_tokens=16, topk=32)
    else:
        model = Pi3SparseLike()
    model = model.to(torch.bfloat16).to(dev).eval()
    g = torch.Generator().manual_seed(4)
    imgs = torch.rand((1, args.frames, 3, hh, ww), generator=g).to(dev)
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
    steps = steps if steps is not None else min(args.steps, 5)
    warmup = warmup if warmup is not None else max(min(args.warmup, 2), 1)
    torch.cuda.reset_peak_memory_stats()
    with torch.no_grad():
        for _ in range(warmup):
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
    tokens = args.frames * (1008 if ref else 1041)
    layout = ("4x4-tile-major patches, no register tokens" if ref else "5 register + 1036 patch per frame")
    bk, tk = (16, 32) if ref else (64, 16)
    res = {
        "metric": "frames/s, Pi3_Sparse-style forward (ViT-L/14 encoder + 36-layer decoder + heads), bf16",
        "value": args.frames / (ms * 1e-3), "unit": "frames/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"cfg5: {args.frames} frames {hh}x{ww} -> {tokens} tokens ({layout}), "
                               f"18 frame-local dense + 18 global sparse attention layers (block {bk}, top-k {tk}), random-init weights",
                   "tokens": tokens, "block": bk, "topk": tk},
        "sparse_attention_ms": sparse_ms, "sparse_attention_share": sparse_ms / ms,
        "sparse_attention_ms_per_layer": sparse_ms / len(model.global_decoder),
        "peak_mem_gb": torch.cuda.max_memory_allocated() / 1e9,
        "outputs": {k: list(v.shape) for k, v in out.items()},
    }
    del model, imgs, out
    torch.cuda.empty_cache()
    return res


def time_layer(step, steps, warmup, overlap, fused):
    """SETTLE_STEPS + `warmup` untimed steps, then exactly `steps` timed ones between two device synchronisations;
    per-kernel spans from HIP events recorded on the launch stream inside every timed step (mean and median)."""
    import statistics

    import torch

    with torch.no_grad():
        for _ in range(SETTLE_STEPS + warmup):
            step()
        torch.cuda.synchronize()
        evs = [{} for _ in range(steps)]
        t0 = time.perf_counter()
        for i in range(steps):
            step(evs[i])
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
    fused = fused and "merge" not in evs[0]   # the merge runs in the selection kernel's epilogue only where that is built
    spans = {}
    if overlap:   # the index kernel runs on a second stream beside the pooling of v and the compressed attention
        spans["pool+compressed_topk (two streams)"] = ("start", "select")
    else:
        spans["pool"] = ("start", "pooled")
        spans["compressed_topk"] = ("pooled", "select")
    if fused:
        spans["select_merge"] = ("select", "end")
    else:
        spans["select"] = ("select", "merge")
        spans["merge"] = ("merge", "end")
    per = {name: [e[a].elapsed_time(e[b]) for e in evs] for name, (a, b) in spans.items()}
    return {"ms_per_step": wall * 1e3 / steps, "fused": fused,
            "mean": {k: sum(v) / len(v) for k, v in per.items()},
            "median": {k: statistics.median(v) for k, v in per.items()}}


def guarded(fn):
    """An extra figure must not take the headline line down with it."""
    try:
        return fn()
    except Exception as exc:  # noqa: BLE001
        return {"error": f"{type(exc).__name__}: {exc}"[:300]}


def _loop_ms(fn, iters=30, settle=20):
    import torch

    for _ in range(settle):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


def hbm_bound_kernels(qd, kd, vd, gd, block, es):
    """GB/s of the memory-bound kernels, each alone on one stream, from their algorithmic bytes: pooling of one tensor,
    the layer's one pass over the packed projection, LayerNorm + RoPE of one tensor, the standalone merge; and, for
    scale, of PyTorch's device-to-device copy of one tensor (``device_copy``: reads and writes 1 : 1, no arithmetic)."""
    import torch

    import speed3r_amd as s3r
    from speed3r_amd.layers import RoPE2D
    from speed3r_amd.sparse_attn import ops

    _, h, n, d = qd.shape
    nc = -(-n // block)
    out = {}
    with torch.no_grad():
        ms = _loop_ms(lambda: s3r.pool_mean(qd, block))
        out["pool"] = (n + nc) * h * d * es / (ms * 1e-3) / 1e9
        out["pool_ms_per_tensor"] = ms
        prepass = _prepass_stage(qd, kd, vd, block)
        ms = _loop_ms(prepass)
        out["prepass"] = ((3 + 2) * n * h * d * es + 3 * nc * h * d * es + n * 2 * 8) / (ms * 1e-3) / 1e9
        out["prepass_ms"] = ms
        del prepass
        t = torch.arange(n, device=qd.device) % 1041
        patch = (t - 5).clamp(min=0)
        pos = torch.where((t >= 5)[:, None], torch.stack((patch // 28 + 1, patch % 28 + 1), dim=-1), torch.zeros_like(t)[:, None])[None]
        cos, sin = RoPE2D(100.0).tables(64, 39, qd.device, qd.dtype)
        w = torch.ones(64, dtype=qd.dtype, device=qd.device)
        ms = _loop_ms(lambda: ops.norm_rope(qd, pos, cos, sin, w, w, 1e-6))
        out["norm_rope"] = 2 * n * h * d * es / (ms * 1e-3) / 1e9
        out["norm_rope_ms"] = ms
        o_cmp = s3r.pool_mean(vd, block)
        ms = _loop_ms(lambda: s3r.gated_merge(o_cmp, vd, gd, block))
        out["merge"] = (2 * n * h * d + n * h * 2 + nc * h * d) * es / (ms * 1e-3) / 1e9
        out["merge_ms"] = ms
        # for scale: PyTorch's device-to-device copy of one tensor (as many bytes written as read, no arithmetic)
        buf = torch.empty_like(qd)
        ms = _loop_ms(lambda: buf.copy_(qd))
        out["device_copy"] = 2 * n * h * d * es / (ms * 1e-3) / 1e9
        del buf
    torch.cuda.empty_cache()
    return out


def run_cfg4(args):
    """The 1000-frame layer (1 041 000 tokens, top-k 16) from the same generator drawn on the device: ms per layer, the
    selection kernel's share of the bf16 MFMA peak and the peak footprint."""
    import torch

    import speed3r_amd as s3r
    from speed3r_amd import workloads

    dev = torch.device("cuda:0")
    cfg = workloads.CONFIGS["cfg4"]
    qd, kd, vd = workloads.make_qkv_on_device(cfg.frames, cfg.dtype, cfg.seed, cfg.low_rank, dev)
    gd = torch.sigmoid(torch.randn((1, 16, cfg.tokens, 2), device=dev, generator=torch.Generator(device=dev).manual_seed(cfg.seed + 1000))).to(cfg.dtype)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()

    def step(timeline=None):
        return s3r.sparse_global_attention(qd, kd, vd, gd, 64, cfg.topk, timeline=timeline)

    global SETTLE_STEPS
    keep, SETTLE_STEPS = SETTLE_STEPS, 10
    try:
        t = time_layer(step, 10, 0, True, True)
    finally:
        SETTLE_STEPS = keep
    sel = t["mean"]["select_merge"]
    res = {"workload": f"{cfg.name}: {cfg.tokens} tokens, 16 heads x 64, block 64, top-k {cfg.topk}, drawn on the device",
           "ms_per_layer": t["ms_per_step"], "kernels_ms": t["mean"], "steps": 10, "settle_steps": 10,
           "select_merge_frac_of_mfma_peak": workloads.selection_flops(cfg.tokens, cfg.topk) / (sel * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
           "effective_tflops": (workloads.selection_flops(cfg.tokens, cfg.topk) + workloads.compressed_flops(cfg.tokens)) / (t["ms_per_step"] * 1e-3) / 1e12,
           "peak_mem_gb": torch.cuda.max_memory_allocated() / 1e9}
    del qd, kd, vd, gd
    torch.cuda.empty_cache()
    return res


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
        print(json.dumps(run_end_to_end(args)))
        return 0
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

    torch.cuda.reset_peak_memory_stats()
    t = time_layer(step, args.steps, args.warmup, overlap, fused)
    peak_mem = torch.cuda.max_memory_allocated()
    ms_per_step, kern_ms, kern_med, fused = t["ms_per_step"], t["mean"], t["median"], t["fused"]
    nc = -(-n // block)
    sel_name = "select_merge" if fused else "select"
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
        "settle_steps": SETTLE_STEPS,
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
        "kernels_median_ms": kern_med,
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
            "frac_of_median_launch": f_sel / (kern_med[sel_name] * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
            # HBM bytes per launch: not measured inside this run; the figure is the one rocprofv3 FETCH_SIZE / WRITE_SIZE
            # gave for this kernel on this workload, scaled by a plain copy (file named in traffic_source, which also
            # names the commit of the kernel it was measured on)
            "traffic": MEASURED_TRAFFIC.get((args.config, topk, block, fused), (None, None))[0],
            "traffic_source": MEASURED_TRAFFIC.get((args.config, topk, block, fused), (None, None))[1],
        },
    }
    headline = args.config == "cfg3" and block == 64 and topk == 16 and not args.no_extras
    if headline:
        t_extras = time.perf_counter()
        result["hbm_gbs"].update(guarded(lambda: hbm_bound_kernels(qd, kd, vd, gd, block, es)))
        del qd, kd, vd, gd
        torch.cuda.empty_cache()
        result["cfg4"] = guarded(lambda: run_cfg4(args))
        if time.perf_counter() - t_extras < 240:
            result["cfg5"] = guarded(lambda: {k2: v2 for k2, v2 in run_end_to_end(args, steps=3, warmup=2).items()
                                              if k2 in ("value", "unit", "ms_per_step", "sparse_attention_share",
                                                        "sparse_attention_ms_per_layer", "peak_mem_gb", "steps", "warmup")})
            if "value" in result["cfg5"]:
                result["cfg5"]["frames_per_s"] = result["cfg5"].pop("value")
        if time.perf_counter() - t_extras < 300:   # the reference model's own setting: 504x392, tile-major, block 16, top-k 32
            result["cfg5_reference_setting"] = guarded(lambda: {
                k2: v2 for k2, v2 in run_end_to_end(args, steps=3, warmup=2, reference_setting=True).items()
                if k2 in ("value", "unit", "ms_per_step", "sparse_attention_share", "sparse_attention_ms_per_layer", "peak_mem_gb")})
            if "value" in result["cfg5_reference_setting"]:
                result["cfg5_reference_setting"]["frames_per_s"] = result["cfg5_reference_setting"].pop("value")
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(q, k, v, gate, block, topk, args.cpu_heads)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
