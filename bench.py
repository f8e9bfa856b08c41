#!/usr/bin/env python3
"""Headline benchmark: Wan-1.3B 480p self-attention SDPA on one MI355X.

One step = one call of the dense SDPA hot path (B=1, H=12, S=32760, d=128, bf16,
scale 1/sqrt(128), non-causal) with Q/K/V already resident in HBM. Prints ONE
JSON line: whole-call TFLOP/s (4*H*Sq*Sk*d FLOPs, the reference's convention,
crates/fastvideo-gpucheck/src/kernels_attn.rs:368), the MFMA roofline of the
flash kernel from HIP-event timings, and the CPU baseline (the fp32 host-math
oracle timed on a bounded sample of query rows, extrapolated to the full call).

Other workloads (--workload cross|causal|causal3|c5|c5cross|tiny|self_d64|vdn32|vsa624|vsa512|prep|layer|kvcache|
kvcache1|composed|softmax) are for the design notes; the driver's line is the default `self`.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "fastvideo-rs_amd"))

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA, published
PEAK_HBM_GBS = 8000.0
# HBM bytes per launch of the flash kernel at the headline workload. NOT measured by this script: the figure
# comes from two rocprofv3 --pmc runs of this same command (FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000 KiB, the
# factors from a plain 1 GiB copy in the same runs), whose summary is the file named beside it.
MEASURED_TRAFFIC_BYTES = {"self": (1.0069e9, "profiles/flash_fwd_pp2_wan13b_self_attention.md")}

WORKLOADS = {
    # name: (H, Sq, Sk, causal block_tokens or 0, description)
    "self": (12, 32760, 32760, 0, "Wan2.1-1.3B 480x832x81 self-attention, B=1 H=12 S=32760 d=128 bf16 non-causal"),
    "cross": (12, 32760, 512, 0, "Wan2.1-1.3B 480p text cross-attention, B=1 H=12 Sq=32760 Sk=512 d=128 bf16"),
    "causal": (12, 32760, 32760, 1560, "Self-Forcing frame-causal, 21 frames x 1560 tokens, H=12 d=128 bf16"),
    "causal3": (12, 32760, 32760, 4680, "Self-Forcing 3-frame blocks (reference geometry), H=12 d=128 bf16"),
    "c5": (40, 75600, 75600, 0, "Wan2.1-14B 720p self-attention, B=1 H=40 S=75600 d=128 bf16"),
    "c5cross": (40, 75600, 512, 0, "Wan2.1-14B 720p cross-attention, H=40 Sq=75600 Sk=512"),
    "tiny": (12, 320, 320, 0, "tiny Wan-1.3B-shaped self-attention, H=12 S=320 d=128"),
    "self_d64": (24, 32760, 32760, 0, "head dim 64 self-attention, B=1 H=24 S=32760 d=64 bf16 non-causal"),
    "vdn32": (12, 49920, 49920, -1, "VDN-H3 window softmax, 32 latent frames x 1560 tokens, chunk 5 radius 1, H=12 d=128"),
}
VDN = (0, 1560, 32, 5, 1)   # video_start, frame_tokens, frames, chunk, radius of the vdn32 workload


VSA_WORKLOADS = {
    # name: (H, grid, sparsity, description)
    "vsa624": (12, (21, 30, 52), 0.8, "VSA, Wan 480p latent grid (21,30,52): 624 tiles, top-k 125, H=12 d=128"),
    "vsa512": (12, (32, 32, 32), 0.875, "VSA, 512 full 4x4x4 cubes (32768 tokens), top-k 64, H=12 d=128"),
}


def bench_vsa(args):
    """Whole VSA op (tile means, coarse scores + top-k, tile pass, block-sparse fine
    kernel, combine) plus each stage alone; FLOPs credited are the fine stage's
    4*(bh*nb*64)*(topk*64)*d, the reference's convention (gpucheck kernels/attn3.rs:747)."""
    import torch

    import fv_sdpa
    from fv_sdpa import vsa as V

    fv_sdpa.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    h, grid, sparsity, desc = VSA_WORKLOADS[args.workload]
    d = 128
    ctx = V.VsaCtx(grid, sparsity, device=dev)
    nb, topk, seq = ctx.num_tiles, ctx.topk, ctx.seq
    g = torch.Generator(device=dev).manual_seed(20241)
    q, k, v, gate = (torch.randn((h, seq, d), generator=g, device=dev).to(torch.bfloat16) for _ in range(4))
    scale = 1.0 / d ** 0.5

    def timed(fn, steps, warmup):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        t0 = time.perf_counter()
        for a, b in evs:
            a.record()
            fn()
            b.record()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) * 1e3 / steps
        ms = sorted(a.elapsed_time(b) for a, b in evs)
        return wall, sum(ms) / len(ms), ms[len(ms) // 2]

    wall, avg_ms, med_ms = timed(lambda: V.vsa_attention_device(q, k, v, gate, ctx, scale), args.steps, args.warmup)
    # stages alone, on the same operands
    qc, kc, vc = (V.vsa_tile_mean(x, ctx) for x in (q, k, v))
    scores, coarse = V.vsa_coarse(qc, kc, vc, scale)
    sel = V.vsa_topk(scores, topk)
    qt, kt, vt = (V.vsa_tile_qkv(x, ctx) for x in (q, k, v))
    sparse = V.vsa_fine(qt, kt, vt, sel, ctx, scale)
    out = torch.empty((h, seq, d), device=dev, dtype=torch.float32)
    stages = {
        "tile_mean_x3": timed(lambda: [V.vsa_tile_mean(x, ctx) for x in (q, k, v)], 10, 2)[2],
        "coarse_scores_softmax_pv": timed(lambda: V.vsa_coarse(qc, kc, vc, scale), 10, 2)[2],
        "topk": timed(lambda: V.vsa_topk(scores, topk), 10, 2)[2],
        "tile_qkv_x3": timed(lambda: [V.vsa_tile_qkv(x, ctx) for x in (q, k, v)], 10, 2)[2],
        "fine": timed(lambda: V.vsa_fine(qt, kt, vt, sel, ctx, scale), 10, 2)[2],
        "combine": timed(lambda: V.vsa_combine(sparse, coarse, gate, ctx, out=out), 10, 2)[2],
    }
    # the whole op on operands a producer already wrote tile-ordered (no tile pass)
    wall_t, avg_t, med_t = timed(lambda: V.vsa_attention_tiled(qt, kt, vt, gate, ctx, scale), args.steps, args.warmup)
    # the fine kernel alone on the selection the reference's own fine-kernel benchmark uses
    # (gpucheck kernels_attn.rs:199-208): tile (i + 7h + j) mod nb for j < topk, i.e. a band of
    # consecutive key tiles that neighbouring query tiles share almost entirely
    ii = torch.arange(nb, device=dev).view(1, nb, 1)
    hh = torch.arange(h, device=dev).view(h, 1, 1)
    jj = torch.arange(topk, device=dev).view(1, 1, topk)
    sel_band = ((ii + 7 * hh + jj) % nb).to(torch.int32).contiguous()
    stages["fine_banded_selection"] = timed(lambda: V.vsa_fine(qt, kt, vt, sel_band, ctx, scale), 10, 2)[2]
    flops = 4.0 * (h * nb * 64) * (topk * 64) * d
    fine_tflops = flops / (stages["fine"] * 1e-3) / 1e12
    rec = {
        "metric": f"VSA TFLOP/s ({args.workload}, fine-stage FLOPs over whole-op time)",
        "value": round(flops / (wall * 1e-3) / 1e12, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(wall, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": desc, "H": h, "grid": list(grid), "tiles": nb, "topk": topk, "seq": seq, "d": d,
                   "inputs": "bf16 q/k/v/gate", "flops_per_call": flops},
        "whole_op_avg_ms": round(avg_ms, 4), "whole_op_median_ms": round(med_ms, 4),
        "whole_op_tile_ordered_inputs_ms": {"avg": round(avg_t, 4), "median": round(med_t, 4), "wall": round(wall_t, 4)},
        "stages_median_ms": {k2: round(v2, 4) for k2, v2 in stages.items()},
        "roofline": {"bound": "mfma", "achieved": round(fine_tflops, 3), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(fine_tflops / PEAK_BF16_TFLOPS, 4), "traffic": None, "kernel": "fv::vsa_fine_kernel<false>",
                     "avg_kernel_ms": round(stages["fine"], 4),
                     "banded_selection_tflops": round(flops / (stages["fine_banded_selection"] * 1e-3) / 1e12, 3)},
    }
    print(json.dumps(rec), flush=True)


def bench_kvcache(args, fpb=3):
    """Autoregressive Self-Forcing self-attention of one layer: blocks of `fpb` latent frames (3: 4680
    tokens, the reference's geometry; 1: 1560 tokens) written into a 21-frame KV cache and each block's
    queries attending the cache window in place (Plan::kv_window). One step = the whole rollout of the
    layer: 21/fpb cache writes + dense calls of Sq = fpb*1560 against Sk = Sq ... 32760, with the keys
    split over several workgroups where the query tiles alone do not fill the GPU (the library's own
    choice, fv_sdpa_splitkv_choose). The same with a contiguous copy of every window first (what the
    reference's `narrow` does) and without split-KV is timed beside it. A rollout is 40 to 90 short
    launches, so each form is captured once as a HIP graph and the replays are timed (what a serving loop
    does); the eager Python loop, whose time depends on the host, is reported beside it."""
    import torch

    import fv_sdpa

    lib = fv_sdpa.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    h, d, ft, frames = 12, 128, 1560, 21
    n, blocks = fpb * ft, frames // fpb
    g = torch.Generator(device=dev).manual_seed(20243)
    qs, ks, vs = ([torch.randn((1, h, n, d), generator=g, device=dev).to(torch.bfloat16) for _ in range(blocks)]
                  for _ in range(3))
    cache = fv_sdpa.CausalKvCache(fv_sdpa.KvSpec.global_window(ft, frames), 1)
    plan = fv_sdpa.Plan.kv_window()
    outs = [torch.empty((h, n, d), device=dev, dtype=torch.bfloat16) for _ in range(blocks)]
    scale = 1.0 / d ** 0.5

    ws_bytes = max(int(lib.fv_sdpa_splitkv_workspace_bytes(h, n, d, 16)), 256)
    ws = torch.empty(ws_bytes, device=dev, dtype=torch.uint8)
    splits_used = []

    def rollout(copy_windows, split=True):
        stream = torch.cuda.current_stream().cuda_stream    # the capturing stream inside a graph capture
        cache.reset()
        for i in range(blocks):
            kw, vw = cache.update(0, ks[i], vs[i], i * n)
            if copy_windows:
                kw, vw = kw.contiguous(), vw.contiguous()
            sk = kw.shape[2]
            rows = kw.stride(1) // d
            sp = int(lib.fv_sdpa_splitkv_choose(h, n, sk)) if split else 1
            if len(splits_used) < blocks and split and not copy_windows:
                splits_used.append(sp)
            rc = lib.fv_sdpa_dense_bf16_splitkv(qs[i].data_ptr(), kw.data_ptr(), vw.data_ptr(), outs[i].data_ptr(), 1,
                                                h, n, sk, d, scale, 0, rows, rows, sp, ws.data_ptr(), ws_bytes, stream)
            if rc != 0:
                raise RuntimeError(lib.fv_sdpa_last_error().decode())

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / args.steps

    def timed_graph(fn):
        fn()                                   # the layer's buffers exist before the capture
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            fn()
        return timed(graph.replay)

    eager = timed(lambda: rollout(False))
    in_place = timed_graph(lambda: rollout(False))
    copied = timed_graph(lambda: rollout(True, split=False))
    unsplit = timed_graph(lambda: rollout(False, split=False))
    # the plan entry once, to show it takes the same route
    kw, vw = cache.update(0, ks[0], vs[0], 0)
    before = fv_sdpa.rt_stats()
    fv_sdpa.sdpa(qs[0], kw, vw, plan)
    assert fv_sdpa.rt_stats()["fused"] == before["fused"] + 1
    flops = sum(4.0 * h * n * (i + 1) * n * d for i in range(blocks))
    tf = flops / (in_place * 1e-3) / 1e12
    rec = {
        "metric": "KV-window attention TFLOP/s (Self-Forcing rollout of one layer, cache read in place)",
        "value": round(tf, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(in_place, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{blocks} blocks x {n} queries against a 21-frame KV cache (Sk = {n} ... 32760), H=12 d=128, "
                               "cache write + attention per block", "flops_per_step": flops,
                   "key_splits_per_block": splits_used},
        "ms_per_step_with_window_copies_no_split": round(copied, 4), "ms_per_step_in_place_no_split": round(unsplit, 4),
        "ms_per_step_eager_python_loop": round(eager, 4),
        "roofline": {"bound": "mfma", "achieved": round(tf, 3), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tf / PEAK_BF16_TFLOPS, 4), "traffic": None, "kernel": "fv::flash_fwd_pp2<false, 128, false, true>"},
    }
    print(json.dumps(rec), flush=True)


def bench_composed(args):
    """The composed f32 SDPA on the device (masked plans, Plan::composed, fallbacks): H=12, S=4096,
    d=128, f32 operands and a shared additive block-causal mask [S, S]; all arithmetic fp32 on the
    matrix cores (v_mfma_f32_32x32x2_f32: 157.3 TFLOP/s peak)."""
    import torch

    import fv_sdpa

    lib = fv_sdpa.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    h, s, d = 12, 4096, 128
    g = torch.Generator(device=dev).manual_seed(20244)
    q, k, v = (torch.randn((h, s, d), generator=g, device=dev) for _ in range(3))
    blk = torch.arange(s, device=dev) // 512
    mask = torch.where(blk[None, :] <= blk[:, None], 0.0, -1e9).to(torch.float32).contiguous()
    out = torch.empty_like(q)
    stream = torch.cuda.current_stream().cuda_stream

    def step():
        rc = lib.fv_sdpa_composed_f32(q.data_ptr(), k.data_ptr(), v.data_ptr(), mask.data_ptr(), 0, out.data_ptr(), h, s,
                                      s, d, 1.0 / d ** 0.5, stream)
        if rc != 0:
            raise RuntimeError(lib.fv_sdpa_last_error().decode())

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    t0 = time.perf_counter()
    for a, b in evs:
        a.record()
        step()
        b.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / args.steps
    avg = sum(a.elapsed_time(b) for a, b in evs) / len(evs)
    flops = 4.0 * h * s * s * d     # every pair is computed (the mask is additive)
    tf = flops / (avg * 1e-3) / 1e12
    rec = {
        "metric": "composed f32 SDPA TFLOP/s (H=12 S=4096 d=128, additive mask)", "value": round(flops / (wall * 1e-3) / 1e12, 3),
        "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "composed f32 SDPA with a shared additive [S, S] mask, H=12 S=4096 d=128", "flops_per_call": flops},
        "roofline": {"bound": "mfma", "achieved": round(tf, 3), "peak": 157.3, "unit": "TFLOP/s", "frac": round(tf / 157.3, 4),
                     "traffic": None, "kernel": "fv::sdpa_composed_mfma_f32_kernel<128>", "avg_kernel_ms": round(avg, 4)},
    }
    print(json.dumps(rec), flush=True)


def bench_prep(args):
    """The producer / consumer either side of the SDPA call at the headline shape: q and k
    RMSNorm + RoPE (bf16 kernel) and the V split out of a fused bf16 QKV projection
    [1, 32760, 3*1536], and merge_heads of the attention output. HBM-bound scans: the
    figure is algorithmic bytes (each operand once) over HIP-event time."""
    import torch

    import fv_sdpa

    fv_sdpa.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    batch, seq, heads, d = 1, 32760, 12, 128
    width = heads * d
    g = torch.Generator(device=dev).manual_seed(20242)
    proj = torch.randn((batch, seq, 3 * width), generator=g, device=dev).to(torch.bfloat16)
    w = (1.0 + 0.1 * torch.randn(width, generator=g, device=dev)).float()
    ang = torch.rand((seq, d // 2), generator=g, device=dev) * 6.0 - 3.0
    cos = torch.cos(ang).repeat_interleave(2, dim=1).contiguous()
    sin = torch.sin(ang).repeat_interleave(2, dim=1).contiguous()
    o = torch.randn((batch, heads, seq, d), generator=g, device=dev).to(torch.bfloat16)

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
        t0 = time.perf_counter()
        for a, b in evs:
            a.record()
            fn()
            b.record()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) * 1e3 / args.steps
        ms = sorted(a.elapsed_time(b) for a, b in evs)
        return wall, sum(ms) / len(ms)

    row = seq * width * 2
    tables = 2 * seq * d * 4
    ops = {
        "qk_norm_rope_bhsd (bf16, rope)": (lambda: fv_sdpa.qk_norm_rope_bhsd(proj, 0, heads, w, (cos, sin)),
                                           2 * row + tables + width * 4),
        "split_heads_bhsd (bf16)": (lambda: fv_sdpa.split_heads_bhsd(proj, 2 * width, heads, d), 2 * row),
        "merge_heads (bf16)": (lambda: fv_sdpa.merge_heads(o), 2 * row),
    }
    # the same producers writing VSA's tile-slot order of the Wan 480p latent grid (21,30,52)
    ctx = fv_sdpa.VsaCtx((21, 30, 52), 0.8, device=dev)
    assert ctx.seq == seq
    qt = torch.zeros((batch, heads, ctx.padded, d), device=dev, dtype=torch.bfloat16)
    vt = torch.zeros_like(qt)
    ops["qk_norm_rope_tiles (bf16, rope)"] = (
        lambda: fv_sdpa.qk_norm_rope_tiles(proj, 0, heads, w, ctx, (cos, sin), out=qt), 2 * row + tables + width * 4)
    ops["split_heads_tiles (bf16)"] = (lambda: fv_sdpa.split_heads_tiles(proj, 2 * width, heads, d, ctx, out=vt), 2 * row)
    res = {}
    for name, (fn, nbytes) in ops.items():
        wall, avg = timed(fn)
        res[name] = {"avg_kernel_ms": round(avg, 4), "ms_per_step": round(wall, 4), "algorithmic_bytes": nbytes,
                     "GBps": round(nbytes / (avg * 1e-3) / 1e9, 1),
                     "frac_of_hbm_peak": round(nbytes / (avg * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)}
    main_op = res["qk_norm_rope_bhsd (bf16, rope)"]
    rec = {
        "metric": "q/k RMSNorm+RoPE -> BHSD GB/s (Wan-1.3B 480p, bf16)", "value": main_op["GBps"], "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": main_op["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "fused QKV projection [1,32760,4608] bf16 -> q/k/v BHSD, H=12 d=128; merge of [1,12,32760,128]"},
        "ops": res,
        "roofline": {"bound": "hbm", "achieved": main_op["GBps"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": main_op["frac_of_hbm_peak"], "traffic": None, "kernel": "fv::qk_norm_rope_bhsd_kernel",
                     "avg_kernel_ms": main_op["avg_kernel_ms"]},
    }
    print(json.dumps(rec), flush=True)


def bench_layer(args):
    """One attention layer's device work at the headline shape, producer to consumer: q and k RMSNorm + RoPE
    (bf16 kernel) and the V split out of a fused bf16 QKV projection [1, 32760, 3*1536], the dense SDPA call,
    merge_heads of its output; timed both ways: the softmax scale applied by the SDPA kernel (scale 1/sqrt(d)),
    and folded into q by the producer (out_mul = scale * log2(e), one float) with the SDPA call at ln 2.
    FLOPs credited are the SDPA call's; the two outputs are compared with each other."""
    import torch

    import fv_sdpa

    lib = fv_sdpa.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    batch, seq, heads, d = 1, 32760, 12, 128
    width = heads * d
    g = torch.Generator(device=dev).manual_seed(20243)
    proj = torch.randn((batch, seq, 3 * width), generator=g, device=dev).to(torch.bfloat16)
    w = (1.0 + 0.1 * torch.randn(width, generator=g, device=dev)).float()
    ang = torch.rand((seq, d // 2), generator=g, device=dev) * 6.0 - 3.0
    cos = torch.cos(ang).repeat_interleave(2, dim=1).contiguous()
    sin = torch.sin(ang).repeat_interleave(2, dim=1).contiguous()
    scale = 1.0 / math.sqrt(d)
    ln2 = 0.6931471805599453
    c = scale * 1.4426950408889634
    flops = 4.0 * heads * seq * seq * d

    def layer(fold):
        q = fv_sdpa.qk_norm_rope_bhsd(proj, 0, heads, w, (cos, sin), out_mul=c if fold else 1.0)
        k = fv_sdpa.qk_norm_rope_bhsd(proj, width, heads, w, (cos, sin))
        v = fv_sdpa.split_heads_bhsd(proj, 2 * width, heads, d)
        o = fv_sdpa.sdpa_dense_bf16(q.reshape(heads, seq, d), k.reshape(heads, seq, d), v.reshape(heads, seq, d),
                                    scale=ln2 if fold else scale, out_bf16=True)
        return fv_sdpa.merge_heads(o.reshape(batch, heads, seq, d))

    def timed(fold):
        for _ in range(args.warmup):
            layer(fold)
        torch.cuda.synchronize()
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
        for a, b in evs:
            a.record()
            layer(fold)
            b.record()
        torch.cuda.synchronize()
        ms = [a.elapsed_time(b) for a, b in evs]
        return sum(ms) / len(ms)

    res = {}
    n0 = lib.fv_sdpa_log2_domain_launches()
    # interleaved, twice each: the clock of the machine drifts by more than the difference looked for
    runs = {False: [], True: []}
    for _ in range(2):
        for fold in (False, True):
            runs[fold].append(timed(fold))
    folded_launches = lib.fv_sdpa_log2_domain_launches() - n0
    assert folded_launches == 2 * (args.warmup + args.steps), folded_launches
    a, b = layer(False).float(), layer(True).float()
    torch.cuda.synchronize()
    diff = (a - b).abs().max().item()
    cos_ab = float((a.flatten().double() @ b.flatten().double()) / (a.double().norm() * b.double().norm()))
    for fold in (False, True):
        ms = sum(runs[fold]) / len(runs[fold])
        res["scale folded into q by the producer" if fold else "scale applied in the SDPA kernel"] = {
            "ms_per_layer": round(ms, 4), "runs_ms": [round(x, 4) for x in runs[fold]],
            "sdpa_tflops_over_layer_time": round(flops / (ms * 1e-3) / 1e12, 1)}
    ms = sum(runs[True]) / len(runs[True])
    rec = {
        "metric": "attention layer (q/k norm+rope, v split, SDPA, merge) ms, Wan-1.3B 480p, bf16", "value": round(ms, 4),
        "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "fused QKV projection [1,32760,4608] bf16 -> q/k/v BHSD -> dense SDPA H=12 S=32760 d=128 -> merge_heads"},
        "forms": res, "max_abs_between_forms": diff, "cosine_between_forms": cos_ab,
    }
    print(json.dumps(rec), flush=True)


def bench_softmax(args):
    """Row softmax entry on score matrices of the shapes the reference materialises: VSA coarse scores
    (12 x 624 rows of 624), a 4096-key chunk, rows of a whole 32760-key call."""
    import torch

    import fv_sdpa

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    shapes = []
    for rows, width in ((12 * 624, 624), (12 * 4096, 4096), (12 * 2048, 8190), (4096, 32760)):
        x = torch.randn((rows, width), device=dev)
        for bf in (False, True):
            out = fv_sdpa.softmax_last(x, out_bf16=bf)
            for _ in range(args.warmup):
                fv_sdpa.softmax_last(x, out_bf16=bf, out=out)
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(args.steps):
                fv_sdpa.softmax_last(x, out_bf16=bf, out=out)
            b.record()
            torch.cuda.synchronize()
            ms = a.elapsed_time(b) / args.steps
            nbytes = rows * width * (4 + (2 if bf else 4))
            shapes.append({"rows": rows, "width": width, "out": "bf16" if bf else "f32", "us": round(ms * 1e3, 2),
                           "GBps": round(nbytes / ms / 1e6, 1)})
        del x, out
    head = shapes[2]
    rec = {
        "metric": "row softmax GB/s (12*4096 rows x 4096, f32 out)", "value": head["GBps"], "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(head["us"] / 1e3, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "fv_softmax_last over f32 score matrices", "shapes": shapes},
        "roofline": {"bound": "hbm", "achieved": head["GBps"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(head["GBps"] / PEAK_HBM_GBS, 4), "traffic": None},
    }
    print(json.dumps(rec), flush=True)


def visible_pairs(sq, sk, bt):
    if bt == 0:
        return sq * sk
    if bt < 0:   # VDN window: frames seen per query frame x frame_tokens^2
        vs, t, frames, c, r = VDN
        total = 0
        for f in range(frames):
            if f in (0, frames - 1):
                seen = frames
            else:
                lo, hi = max(0, (f // c - r) * c), min(frames - 1, (f // c + r + 1) * c - 1)
                seen = len(set(range(lo, hi + 1)) | {0, frames - 1})
            total += seen * t * t
        return total
    total = 0
    for qb in range((sq + bt - 1) // bt):
        nq = min(bt, sq - qb * bt)
        total += nq * min(sk, (qb + 1) * bt)
    return total


def cpu_baseline(h, sq, sk, d, bt, flops_full, q, k, v, budget_s, gpu_out=None, scale=None):
    """Time the oracle's fp32 composed SDPA on a bounded sample of query rows; with `gpu_out` (the
    kernel's output of the timed launches) also compare those rows, all heads, with the oracle's."""
    import numpy as np

    import oracle

    cores = os.cpu_count() or 1
    threads = max(1, min(h, cores, 16))
    qn, kn, vn = (x.float().cpu().numpy() for x in (q, k, v))
    mask = (bt, 0, 0) if bt else None
    rng = np.random.Generator(np.random.PCG64(7))

    def run(n):
        rows = np.sort(rng.choice(sq, size=min(n, sq), replace=False)).astype(np.int64)
        t0 = time.perf_counter()
        want = oracle.sdpa_composed_rows(qn, kn, vn, rows, scale=scale, mask_bc=mask, threads=threads)
        return time.perf_counter() - t0, rows, want

    t_probe, rows, _ = run(min(16, sq))
    per_row = max(t_probe / rows.size, 1e-9)
    t, rows, want = run(int(max(rows.size, min(sq, budget_s / per_row))))
    n = rows.size
    t_full = t * sq / n
    parity = None
    if gpu_out is not None:
        import torch

        got = gpu_out[:, torch.from_numpy(rows).to(gpu_out.device)].float().cpu().numpy().astype(np.float64)
        w64 = want.astype(np.float64)
        parity = {"rows": int(n), "heads": int(h), "max_abs": float(np.abs(got - w64).max()),
                  "cosine": float((got.ravel() @ w64.ravel()) / (np.linalg.norm(got) * np.linalg.norm(w64))),
                  "tolerance": "max_abs <= 1e-2, cosine >= 0.9999 vs the fp32 host-math oracle",
                  "finite": bool(np.isfinite(got).all())}
        parity["ok"] = bool(parity["finite"] and parity["max_abs"] <= 1e-2 and parity["cosine"] >= 0.9999)
    return parity, {
        "value": flops_full / t_full / 1e12,
        "unit": "TFLOP/s",
        "cores": threads,
        "kind": "port",
        "sample": f"{n} of {sq} query rows x all {h} heads x all {sk} keys in {t:.2f} s, "
                  f"extrapolated x{sq / n:.1f} to {t_full:.1f} s/call; host has {cores} cores, "
                  f"threads split heads only (as the reference's rayon matmul)",
        "ms_per_call_extrapolated": t_full * 1e3,
    }


def lib_is_log2_domain(lib, scale):
    return lib.fv_sdpa_is_log2_domain_scale(scale) == 1


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=8,
                    help="untimed launches first; the shader clock under this kernel takes about six launches to settle")
    ap.add_argument("--workload", default="self", choices=sorted(WORKLOADS) + sorted(VSA_WORKLOADS) + ["prep", "layer", "kvcache", "kvcache1", "composed", "softmax"])
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="CPU baseline sample budget; 0 skips it")
    ap.add_argument("--out-bf16", type=int, default=1)
    ap.add_argument("--inputs", default="randn", choices=["randn", "zeros"],
                    help="attention workloads only. zeros: the same launches on all-zero Q/K/V, a power experiment "
                         "(same instruction stream, no bit activity in the operands); never the headline")
    ap.add_argument("--fold-scale", type=int, default=0,
                    help="attention workloads only. 1: Q is drawn as bf16(N(0,1) * scale * log2 e) and the call passes "
                         "scale = ln 2, what a caller that folds the softmax scale into the q RMSNorm weight does; the "
                         "kernels then run their form without the per-score multiply-add; never the headline")
    ap.add_argument("--copy-calibration-mib", type=int, default=0,
                    help="also launch one plain device copy of this many MiB (known HBM traffic, to scale "
                         "profiler byte counters); not part of the timed region")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs the full sequence on ONE GPU (no sharding, no collectives); "
              "--gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import torch

    import fv_sdpa

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(3)
    if args.workload in VSA_WORKLOADS:
        bench_vsa(args)
        return
    if args.workload == "prep":
        bench_prep(args)
        return
    if args.workload in ("kvcache", "kvcache1"):
        bench_kvcache(args, 3 if args.workload == "kvcache" else 1)
        return
    if args.workload == "layer":
        bench_layer(args)
        return
    if args.workload == "composed":
        bench_composed(args)
        return
    if args.workload == "softmax":
        bench_softmax(args)
        return
    fv_sdpa.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    h, sq, sk, bt, desc = WORKLOADS[args.workload]
    d = 64 if args.workload.endswith("_d64") else 128
    g = torch.Generator(device=dev).manual_seed(20240)
    scale = 1.0 / d ** 0.5
    q = torch.randn((h, sq, d), generator=g, device=dev)
    if args.fold_scale:
        q *= scale * 1.4426950408889634
        scale = float(torch.tensor(math.log(2.0), dtype=torch.float32).item())
        if not lib_is_log2_domain(fv_sdpa.lib(), scale):
            raise RuntimeError("scale = ln 2 does not select the log2-domain form")
    q = q.to(torch.bfloat16)
    k = torch.randn((h, sk, d), generator=g, device=dev).to(torch.bfloat16)
    v = torch.randn((h, sk, d), generator=g, device=dev).to(torch.bfloat16)
    if args.inputs == "zeros":
        q.zero_(), k.zero_(), v.zero_()
    out = torch.empty((h, sq, d), device=dev, dtype=torch.bfloat16 if args.out_bf16 else torch.float32)
    lib = fv_sdpa.lib()
    stream = torch.cuda.current_stream().cuda_stream

    def step():
        if bt < 0:
            rc = lib.fv_sdpa_vdn_window_bf16(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                             args.out_bf16, h, sq, sk, d, scale, *VDN, stream)
        elif bt:
            rc = lib.fv_sdpa_block_causal_bf16(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                               args.out_bf16, h, sq, sk, d, scale, bt, 0, 0, stream)
        else:
            rc = lib.fv_sdpa_dense_bf16(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                        args.out_bf16, h, sq, sk, d, scale, stream)
        if rc != 0:
            raise RuntimeError(f"kernel rc={rc}: {lib.fv_sdpa_last_error().decode()}")

    if args.copy_calibration_mib > 0:
        src = torch.empty(args.copy_calibration_mib << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)   # one elementwise copy kernel: reads and writes exactly this many bytes
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # whole-region wall clock, bracketed by synchronisation on both sides
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    t0 = time.perf_counter()
    for a, b in evs:
        a.record()
        step()
        b.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    kern_ms = sorted(a.elapsed_time(b) for a, b in evs)
    avg_kernel_ms = sum(kern_ms) / len(kern_ms)
    ms_per_step = wall * 1e3 / args.steps

    flops = 4.0 * h * visible_pairs(sq, sk, bt) * d
    flops_dense_equiv = 4.0 * h * sq * sk * d
    value = flops / (ms_per_step * 1e-3) / 1e12
    achieved = flops / (avg_kernel_ms * 1e-3) / 1e12
    bytes_min = 2.0 * (2 * h * sq * d + 2 * h * sk * d)

    traffic, traffic_source = MEASURED_TRAFFIC_BYTES.get(args.workload, (None, None)) if args.out_bf16 else (None, None)
    if traffic_source:
        traffic_source += " (rocprofv3 --pmc runs of this command; not measured in this run)"
    rec = {
        "metric": "SDPA TFLOP/s + % bf16 MFMA peak, Wan-1.3B 480p self-attn (S=32760,H=12,d=128)"
        if args.workload == "self" and not args.fold_scale else
        f"SDPA TFLOP/s ({args.workload}{', softmax scale folded into Q' if args.fold_scale else ''})",
        "value": round(value, 3),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": ("synthetic" if args.inputs == "randn" else "all-zero operands (power experiment, not a benchmark)") +
                (" (Q = bf16(N(0,1) * scale * log2 e), call scale ln 2)" if args.fold_scale else ""),
        "config": {"workload": desc, "H": h, "Sq": sq, "Sk": sk, "d": d, "block_tokens": bt,
                   "out": "bf16" if args.out_bf16 else "f32", "flops_per_call": flops,
                   "dense_equivalent_flops": flops_dense_equiv},
        "pct_of_bf16_mfma_peak": round(100.0 * value / PEAK_BF16_TFLOPS, 2),
        "roofline": {"bound": "mfma", "achieved": round(achieved, 3), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
                     "traffic": traffic, "traffic_source": traffic_source,
                     # template arguments: masked, head dim, scale folded into Q, fixed-offset first pass (launches
                     # that write bf16 and whose queries all see key 0: every workload here)
                     "kernel": f"fv::flash_fwd_pp2<{'true' if bt else 'false'}, {d}, {'true' if args.fold_scale else 'false'}, "
                               f"{'true' if args.out_bf16 and os.environ.get('FASTVIDEO_SDPA_RUNNING_MAX', '0') in ('', '0') else 'false'}>",
                     "avg_kernel_ms": round(avg_kernel_ms, 4), "median_kernel_ms": round(kern_ms[len(kern_ms) // 2], 4),
                     "min_hbm_bytes": bytes_min,
                     "hbm_frac_at_min_traffic": round(bytes_min / (avg_kernel_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)},
    }
    if args.cpu_seconds > 0 and bt >= 0:   # the row-sampled oracle takes dense and block-causal masks
        # outside the timed region; the rows the baseline computes double as a parity sample of this run's output
        parity, rec["cpu_baseline"] = cpu_baseline(h, sq, sk, d, bt, flops, q, k, v, args.cpu_seconds,
                                                   out if args.inputs == "randn" else None,
                                                   scale if args.fold_scale else None)
        if parity is not None:
            rec["parity"] = parity
    print(json.dumps(rec), flush=True)
    if rec.get("parity") is not None and not rec["parity"]["ok"]:
        print("bench.py: the timed launches' output is outside the parity tolerance", file=sys.stderr)
        sys.exit(5)


if __name__ == "__main__":
    main()
