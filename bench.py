#!/usr/bin/env python3
"""Benchmark of the MoE expert-layer hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 1]

A step is one forward pass of the layer (router -> permute+quant -> gate_up/SwiGLU/
requant GEMM -> down GEMM -> combine + shared expert) over one batch of synthetic
tokens, with weights and inputs already resident in HBM.  The default run prints ONE JSON line for
configuration 1 of the benchmark set (DeepSeek-V3-shaped FP8 decode, 256 tokens, 32 of 256 experts local, masked
layout: the HBM GB/s half of the metric) whose `prefill` object holds configuration 2 (the same layer on 16384
tokens, ragged layout: the FP8 TFLOP/s half), each with its roofline and CPU baseline.  `--config N` measures one
configuration only.  Decode configurations are also timed with 512 MiB read through the chip before every pass
(`cache_flushed`), so that nothing of the previous pass is left in the 256 MiB last-level cache.

`--op router_gemm` and `--op norm_quant` time the two producers that sit in front of the layer on the same
configuration's shapes (hidden states -> logits -> routes in two launches; residual add + RMSNorm + FP8
cast in one) and print the same kind of line for them.  `--op dense_expert [--rows R]` times the dense FP8 expert
chain (the shared expert as the reference's model code runs it outside the grouped launch).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0          # MI355X published HBM3E bandwidth
FP8_PEAK_TFLOPS = 5000.0        # MI355X published dense FP8 MFMA peak
BF16_PEAK_TFLOPS = 2500.0       # MI355X published dense BF16 MFMA peak

METRIC = "MoE layer TFLOP/s (FP8 prefill) & HBM GB/s (decode), % roofline, 1xMI355X"

MIB = 1024 * 1024
FLUSH_BYTES = 512 * MIB         # read between flushed replays: twice the 256 MiB last-level (Infinity) cache
DEVICE = "cuda:0"               # the one GPU this benchmark runs on


def traffic_record(key):
    """HBM bytes per launch of a dominant kernel, as measured with `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE`
    (each scaled by what the counter reads for a plain copy kernel of known size in the same run).  The figures
    live in the summaries under profiles/, each in a line `traffic-record: {json}` that names the workload
    (`key`), the bytes, the git commit of the measurement and the SHA-256 of every kernel source file the
    measured kernel is built from.  A record is used only while those files are unchanged: a figure measured on
    another version of the kernel says nothing about this one, and null is reported instead."""
    import glob
    import hashlib
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*.md"))):
        for line in open(path, encoding="utf-8"):
            if "traffic-record:" not in line:
                continue
            try:
                rec = json.loads(line.split("traffic-record:", 1)[1].strip().rstrip("->").strip())
            except ValueError:
                continue
            if str(rec.get("key")) != str(key):
                continue
            for rel, want in rec.get("sources", {}).items():
                try:
                    got = hashlib.sha256(open(os.path.join(ROOT, rel), "rb").read()).hexdigest()
                except OSError:
                    got = None
                if got != want:
                    then = (int(rec["fetch_bytes"]) + int(rec["write_bytes"])) / 1e6
                    return None, (f"{os.path.basename(path)}: {rel} changed since the measurement (commit "
                                  f"{rec.get('commit')}, which read {then:.1f} MB per launch)")
            return int(rec["fetch_bytes"]) + int(rec["write_bytes"]), f"{os.path.basename(path)} (commit {rec.get('commit')})"
    return None, "no record under profiles/"


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", type=int, default=None, choices=[0, 1, 2, 3, 4, 5],
                    help="0-4: the benchmark set's configurations; 5: the Kimi-K3 latent MoE layer at its real shape. "
                         "Default: configuration 1 (decode) as the line, plus configuration 2 (prefill) in its "
                         "`prefill` object -- the two halves of the metric")
    ap.add_argument("--op", default="layer", choices=["layer", "router_gemm", "norm_quant", "dense_expert"],
                    help="what one step is: the MoE layer (default), one of its two producers, or the dense FP8 "
                         "expert chain (the shared expert outside the grouped launch) on the configuration's shapes")
    ap.add_argument("--rows", type=int, default=0, help="--op dense_expert: rows per step (default: the "
                                                        "configuration's token count)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--dense-backend", default=None, choices=["hip", "vendor"],
                    help="MXFP4 configurations: the bf16 shared expert and latent projections on this library's "
                         "bf16 GEMM (hip, the layer's default) or on the vendor library through torch.mm (vendor)")
    ap.add_argument("--graph", action="store_true",
                    help="time replays of one captured HIP graph of the layer instead of eager launches")
    ap.add_argument("--tiled-variant", type=int, default=0, choices=[0, 1, 2],
                    help="which LDS-tiled kernel serves the prefill groups: 0 = K steps of 128 (default), 1 = K steps of "
                         "64 with in-place accumulation, 2 = the same with plain per-lane stores (bgmoe_set_tiled_variant)")
    ap.add_argument("--mxfp4-variant", type=int, default=0, choices=[0, 1, 2, 3],
                    help="MXFP4 configurations: 0 = 64-row items with three prefetch stages (default), 1 = 32-row items "
                         "with six, 2 = per group: 32-row items (five stages) up to 32 rows, 64-row items above, 3 = 64-row items with four "
                         "(bgmoe_set_mxfp4_variant)")
    ap.add_argument("--bf16-gemm-plan", type=int, default=-1, choices=[-1, 0, 1, 2, 3, 4, 5],
                    help="launch shape of the bf16 GEMM behind the router GEMM and the MXFP4 layers' linear layers "
                         "(bgmoe_set_router_gemm_plan(-1, plan)): -1 = chosen from the sizes (default), 5 = 128 x 64 tiles")
    ap.add_argument("--fold-gather", action="store_true",
                    help="MXFP4 configurations: stage 1 reads its rows from the tokens through the dispatch's row -> pair "
                         "map instead of from a gathered copy (Mxfp4MoELayer(fold_gather=True))")
    ap.add_argument("--tall-min-rows", type=int, default=0,
                    help="decode: groups with more rows than this run as 64-row stage-1 items of the weight-streaming "
                         "kernel (bgmoe_set_skinny_tall_min_rows; 0 = off, the default)")
    ap.add_argument("--gemm-stages", type=int, default=2, choices=[2, 3, 4, 6],
                    help="decode: prefetch depth of the weight-streaming down projection "
                         "(bgmoe_set_skinny_gemm_stages; 2 = the default)")
    ap.add_argument("--s1-stages", type=int, default=3, choices=[3, 4],
                    help="decode: prefetch depth of the weight-streaming fused stage 1 (bgmoe_set_skinny_s1_stages; "
                         "3 = the default)")
    ap.add_argument("--template", action="store_true",
                    help="FP8 configurations: also time the layer as a model file runs it through the MoEBase template "
                         "(router GEMM + gate, routed experts behind the given routes, dense shared expert, add) and "
                         "report it as `template_layer` next to the one-call layer")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch one plain copy kernel of known size (the weight re-layout kernel on a "
                         "256 MiB buffer: 256 MiB read, 256 MiB written) so that rocprofv3 --pmc FETCH_SIZE / "
                         "WRITE_SIZE readings can be scaled")
    return ap.parse_args()


def cpu_baseline(cfg, inp, w, sh, ids, wt, alg_bytes, flops):
    """The reference's CPU-runnable PyTorch path (oracle.layer.moe_layer_l1_torch) on the host cores."""
    import numpy as np
    import torch
    from oracle import layer as ol

    cores = os.cpu_count() or 1
    threads = min(cores, 16)
    torch.set_num_threads(threads)

    def deq(q, s):     # deepseek_v3_dequantization -> bf16, per expert to bound memory
        n, k = q.shape[-2:]
        v = q.to(torch.float32).view(n // 128, 128, k // 128, 128) * s[:, None, :, None]
        return v.view(n, k).to(torch.bfloat16)

    # bounded sample: at most 8192 tokens and the experts those tokens use
    n = min(cfg.n_tokens, 8192)
    x = inp["x"][:n].cpu()
    ids_n, wt_n = ids[:n], wt[:n]
    used = np.unique(ids_n)
    experts = []
    for e in range(cfg.e_local):
        if (e + cfg.expert_start) in used:
            experts.append(tuple(deq(w[k + "_q"][e].cpu(), w[k + "_s"][e].cpu()) for k in ("gate", "up", "down")))
        else:
            experts.append(None)
    shared = None
    if sh is not None:
        shared = tuple(deq(sh[k + "_q"][0].cpu(), sh[k + "_s"][0].cpu()) for k in ("gate", "up", "down"))
    dummy = torch.zeros(1, 1, dtype=torch.bfloat16)
    experts = [e if e is not None else (dummy, dummy, dummy) for e in experts]
    reps = 3
    ol.moe_layer_l1_torch(x, ids_n, wt_n, experts, cfg.expert_start, shared)
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        ol.moe_layer_l1_torch(x, ids_n, wt_n, experts, cfg.expert_start, shared)
        ts.append(time.perf_counter() - t0)
    t = sorted(ts)[len(ts) // 2]
    frac = n / cfg.n_tokens
    return t, threads, cores, f"{n} of {cfg.n_tokens} tokens of the workload, all experts they route to, " \
                              f"bf16 dequantised weights, 1 warm-up + median of {reps}", frac


def cpu_baseline_mxfp4(cfg, inp, w, sh, lat=None):
    """The NumPy restatement of the MXFP4 layer (oracle.layer.moe_layer_mxfp4: dequantise, bf16-valued GEMMs,
    SwiGLU, combine) on a few tokens; its cost is dominated by dequantising the experts those tokens use."""
    import torch
    from oracle import layer as ol
    n = min(cfg.n_tokens, 8)
    wn = {k: v.cpu().numpy() for k, v in w.items()}
    shn = {k: v.float().cpu().numpy() for k, v in sh.items()} if sh else None
    t0 = time.perf_counter()
    ol.moe_layer_mxfp4(inp["x"][:n].cpu(), inp["logits"][:n].cpu().numpy(), inp["bias"].cpu().numpy(),
                       dict(top_k=cfg.top_k, n_group=1, topk_group=1, rsf=cfg.rsf), wn, cfg.expert_start,
                       cfg.e_local, layout="masked", max_tokens=cfg.max_tokens, shared_bf16=shn,
                       activation=cfg.activation,
                       latent=None if lat is None else {k: (v.cpu() if torch.is_tensor(v) else v) for k, v in lat.items()})
    t = time.perf_counter() - t0
    return t, n / cfg.n_tokens, f"{n} of {cfg.n_tokens} tokens of the workload and the experts they route to, one pass, NumPy"


def _time(step, steps, warmup, torch):
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        step()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps


def bench_producer(a):
    """One step = the router GEMM + top-k, or the add + RMSNorm + FP8 cast, on the configuration's shapes."""
    import numpy as np
    import torch
    from batchgen_amd import _lib, workloads as wl
    dev = torch.device(DEVICE)
    torch.cuda.set_device(dev)
    if a.config is None:
        a.config = 1
    cfg = wl.CONFIGS[a.config]
    n, h, e, k = cfg.n_tokens, cfg.hidden, cfg.n_experts, cfg.top_k
    g = torch.Generator(device=dev).manual_seed(cfg.seed + 7)
    base = {"n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "launch": "eager", "data": "synthetic"}
    if a.copy_calibration:
        from batchgen_amd.moe.fp8_layer import repack_tile_major
        repack_tile_major(torch.zeros((1, 32768, 8192), dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn))
        torch.cuda.synchronize()
    if a.op == "router_gemm":
        from batchgen_amd.moe.routing import router_gemm_gate_sigmoid_topk
        x = (torch.randn(n, h, generator=g, device=dev) * 0.1).to(torch.bfloat16)
        w = (torch.randn(e, h, generator=g, device=dev) * 0.1).to(torch.bfloat16)
        bias = torch.zeros(e, device=dev)
        ids = torch.empty((n, k), dtype=torch.int32, device=dev)
        wt = torch.empty((n, k), dtype=torch.float32, device=dev)
        grouped = cfg.n_group > 1
        step = lambda: router_gemm_gate_sigmoid_topk(x, w, bias, k, cfg.rsf, ids, wt,
                                                     n_group=cfg.n_group if grouped else 0,
                                                     topk_group=cfg.topk_group if grouped else 0)
        ms = _time(step, a.steps, a.warmup, torch)
        _lib.prof_enable(True)
        for _ in range(a.steps):
            step()
        prof = _lib.prof_collect()
        _lib.prof_enable(False)
        gemm_ms = prof["router_gemm"][0] / prof["router_gemm"][1]
        flops = 2.0 * n * h * e
        alg_bytes = (n + e) * h * 2 + n * k * 8
        mfma = flops / (BF16_PEAK_TFLOPS * 1e12) > alg_bytes / (HBM_PEAK_GBPS * 1e9)
        if mfma:
            roof = dict(bound="mfma", kernel="router_gemm_kernel", achieved=flops / (gemm_ms * 1e-3) / 1e12,
                        peak=BF16_PEAK_TFLOPS, unit="TFLOP/s", traffic=None, flops_per_launch=flops,
                        avg_launch_us=gemm_ms * 1e3)
        else:
            gb = (n + e) * h * 2
            roof = dict(bound="hbm", kernel="router_gemm_kernel", achieved=gb / (gemm_ms * 1e-3) / 1e9,
                        peak=HBM_PEAK_GBPS, unit="GB/s", traffic=None, bytes_per_launch=gb,
                        avg_launch_us=gemm_ms * 1e3)
        roof["frac"] = roof["achieved"] / roof["peak"]
        roof["traffic"], roof["traffic_source"] = traffic_record(f"{a.op}:{a.config}")
        out = dict(base, metric="router GEMM + top-k: TFLOP/s (prefill) or HBM GB/s (decode), 1xMI355X",
                   value=(flops / (ms * 1e-3) / 1e12) if mfma else (alg_bytes / (ms * 1e-3) / 1e9),
                   unit="TFLOP/s" if mfma else "GB/s", ms_per_step=ms, dtype="bf16 (fp32 accumulate)",
                   config={"workload": cfg.name + " / router", "tokens": n, "hidden": h, "experts": e, "top_k": k},
                   tokens_per_s=n / (ms * 1e-3), kernel_ms_per_step={kk: v[0] / a.steps for kk, v in prof.items()},
                   roofline=roof)
        if not a.no_cpu_baseline:
            from oracle import router as orr               # the CPU port is the baseline leg only
            from oracle import router_gemm as org
            m = min(n, 512)
            xs, wc = x[:m].cpu(), w.cpu()
            t0 = time.perf_counter()
            logits = org.router_gemm_exact(xs, wc)
            if grouped:
                orr.grouped_router(logits, bias.cpu().numpy(), cfg.n_group, cfg.topk_group, k, cfg.rsf)
            else:
                orr.gate_sigmoid_topk(logits, bias.cpu().numpy(), k, cfg.rsf)
            t = time.perf_counter() - t0
            frac = m / n
            out["cpu_baseline"] = {"value": (flops * frac / t / 1e12) if mfma else (alg_bytes * frac / t / 1e9),
                                   "unit": out["unit"], "cores": min(os.cpu_count() or 1, 16), "kind": "port",
                                   "sample": f"{m} of {n} tokens, float64 BLAS product + NumPy router", "seconds": t}
        print(json.dumps(out))
        return
    if a.op == "dense_expert":
        return bench_dense_expert(a, cfg, dev, g, base)
    res = (torch.randn(n, h, generator=g, device=dev) * 0.9).to(torch.bfloat16)
    hid = (torch.randn(n, h, generator=g, device=dev) * 0.4).to(torch.bfloat16)
    gamma = (torch.randn(h, generator=g, device=dev) * 0.3 + 1.0).to(torch.bfloat16)
    res0 = res.clone()
    from batchgen_amd._lib import check, lib, ptr, stream
    normed = torch.empty_like(res)
    q = torch.empty((n, h), dtype=torch.uint8, device=dev)
    sc = torch.empty((n, h // 128), dtype=torch.float32, device=dev)
    # the residual is updated in place; its growth over the timed steps does not change the work done
    step = lambda: check(lib().bgmoe_add_rmsnorm_fp8_quant(ptr(res), ptr(hid), ptr(gamma), n, h, 1e-5, ptr(normed),
                                                           ptr(q), ptr(sc), h // 128, 1, None, None, None, stream()))
    ms = _time(step, a.steps, a.warmup, torch)
    _lib.prof_enable(True)
    for _ in range(a.steps):
        step()
    prof = _lib.prof_collect()
    _lib.prof_enable(False)
    k_ms = prof["norm_quant"][0] / prof["norm_quant"][1]
    alg_bytes = n * h * 9 + n * (h // 128) * 4 + h * 2
    roof = dict(bound="hbm", kernel="add_rmsnorm_fp8_quant_kernel", achieved=alg_bytes / (k_ms * 1e-3) / 1e9,
                peak=HBM_PEAK_GBPS, unit="GB/s", traffic=None, bytes_per_launch=alg_bytes, avg_launch_us=k_ms * 1e3)
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["traffic"], roof["traffic_source"] = traffic_record(f"{a.op}:{a.config}")
    out = dict(base, metric="add + RMSNorm + FP8 cast: HBM GB/s, 1xMI355X", value=alg_bytes / (ms * 1e-3) / 1e9,
               unit="GB/s", ms_per_step=ms, dtype="bf16 in, fp32 arithmetic, e4m3 + fp32 scales out",
               config={"workload": cfg.name + " / add_rmsnorm_fp8_quant", "rows": n, "hidden": h},
               tokens_per_s=n / (ms * 1e-3), roofline=roof)
    if not a.no_cpu_baseline:
        from oracle import norm_quant as onq               # the CPU port is the baseline leg only
        m = min(n, 256)
        t0 = time.perf_counter()
        onq.add_rmsnorm_fp8_quant(res0[:m].cpu(), hid[:m].cpu(), gamma.cpu(), 1e-5)
        t = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": alg_bytes * (m / n) / t / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": f"{m} of {n} rows, NumPy oracle, one thread", "seconds": t}
    print(json.dumps(out))


def bench_dense_expert(a, cfg, dev, g, base):
    """One step = quantise(x) -> [gate; up] GEMM -> SiLU * up + quantise -> down GEMM of ONE dense FP8 expert
    (hidden x shared_inter of the configuration) on `rows` rows."""
    import numpy as np
    import torch
    from batchgen_amd import _lib
    from batchgen_amd.moe.shared_expert import Fp8DenseExpert
    rows = a.rows or cfg.n_tokens
    h, inter = cfg.hidden, cfg.shared_inter or cfg.inter

    def fp8_weight(n, k):
        q = (torch.randn(n, k, generator=g, device=dev) * 64).to(torch.float8_e4m3fn)
        sc = torch.rand(n // 128, k // 128, generator=g, device=dev) * 2e-4 + 1e-4
        return q, sc
    gate_up, gu_s = fp8_weight(2 * inter, h)
    down, d_s = fp8_weight(h, inter)
    expert = Fp8DenseExpert(gate_up[:inter], gu_s[:inter // 128].contiguous(), gate_up[inter:],
                            gu_s[inter // 128:].contiguous(), down, d_s, gate_up=gate_up)
    x = (torch.randn(rows, h, generator=g, device=dev) * 0.5).to(torch.bfloat16)
    out_buf = torch.empty(rows, h, dtype=torch.bfloat16, device=dev)
    step = lambda: expert(x, out=out_buf)
    if a.graph:                                  # replays of one captured chain: what a serving loop runs
        for _ in range(3):
            step()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        ms = _time(graph.replay, a.steps, a.warmup, torch)
        base = dict(base, launch="hip_graph")
    else:
        ms = _time(step, a.steps, a.warmup, torch)
    _lib.prof_enable(True)
    for _ in range(a.steps):
        step()
    prof = _lib.prof_collect()
    _lib.prof_enable(False)
    key = "fp8_dense_gemm" if "fp8_dense_gemm" in prof else "gemm_skinny16"
    k_ms = prof[key][0] / prof[key][1]                       # average over the chain's two GEMMs
    w_bytes = 3 * inter * h + (3 * inter * h // 16384) * 4
    alg_bytes = w_bytes + rows * h * 2 * 2                   # weights once, bf16 rows in and out
    gemm_bytes = w_bytes / 2                                 # per GEMM launch, averaged like k_ms
    roof = dict(bound="hbm", kernel=key + " (average of the chain's gate_up and down GEMMs)",
                achieved=gemm_bytes / (k_ms * 1e-3) / 1e9, peak=HBM_PEAK_GBPS, unit="GB/s", traffic=None,
                bytes_per_launch=gemm_bytes, avg_launch_us=k_ms * 1e3)
    roof["frac"] = roof["achieved"] / roof["peak"]
    out = dict(base, metric="dense FP8 expert chain: HBM GB/s over its algorithmic bytes, 1xMI355X",
               value=alg_bytes / (ms * 1e-3) / 1e9, unit="GB/s", ms_per_step=ms,
               dtype="e4m3 x e4m3 -> fp32, bf16 in and out",
               config={"workload": cfg.name + " / dense_expert", "rows": rows, "hidden": h, "intermediate": inter},
               tokens_per_s=rows / (ms * 1e-3), kernel_ms_per_step={kk: v[0] / a.steps for kk, v in prof.items()},
               roofline=roof)
    if not a.no_cpu_baseline:
        from oracle import gemm as og                        # the CPU port is the baseline leg only
        from oracle import quant as oq
        m = min(rows, 32)
        one = np.array([m], np.int32), np.array([0, m], np.int32)
        gq, gs = gate_up.cpu().view(torch.uint8).numpy()[None], gu_s.cpu().numpy()[None]
        dq, ds = down.cpu().view(torch.uint8).numpy()[None], d_s.cpu().numpy()[None]
        t0 = time.perf_counter()
        xq, xs = oq.act_quant(x[:m].float().cpu().numpy(), form="A")
        gu = og.grouped_gemm_fp8(xq, xs, gq, gs, *one)
        hq, hs, _ = oq.silu_mul_group_quant(gu[:, :inter], gu[:, inter:], "A")
        og.grouped_gemm_fp8(hq, hs, dq, ds, *one)
        t = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": alg_bytes / t / 1e9, "unit": "GB/s", "cores": min(os.cpu_count() or 1, 16),
                               "kind": "port", "sample": f"{m} of {rows} rows, NumPy oracle chain (weights "
                               "dequantised once per call, as the algorithmic bytes count them)", "seconds": t}
    print(json.dumps(out))


def cpu_baseline_mxfp4_torch(cfg, inp, w, sh, ids, wt):
    """The reference's CPU-runnable PyTorch path on MXFP4 experts: weights dequantised to bf16 with the reference
    recipe (oracle.layer.l1_dequant_mxfp4, batchgen/moe/mxfp4_oracle_vector.py:80-115), then the same per-expert
    bf16 loop as the FP8 baseline (oracle.layer.moe_layer_l1_torch).  Latent configurations are not covered by that
    loop and keep the NumPy pass."""
    import numpy as np
    import torch
    from oracle import layer as ol
    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    n = min(cfg.n_tokens, 128)
    ids_n, wt_n = ids[:n], wt[:n]
    used = np.unique(ids_n)
    dummy = torch.zeros(1, 1, dtype=torch.bfloat16)
    experts = []
    for e in range(cfg.e_local):
        if (e + cfg.expert_start) in used:
            experts.append(tuple(ol.l1_dequant_mxfp4(w[k + "_p"][e].cpu().numpy(), w[k + "_s"][e].cpu().numpy())
                                 for k in ("gate", "up", "down")))
        else:
            experts.append((dummy, dummy, dummy))
    shared = tuple(sh[k].cpu() for k in ("gate", "up", "down")) if sh else None
    x = inp["x"][:n].cpu()
    ol.moe_layer_l1_torch(x, ids_n, wt_n, experts, cfg.expert_start, shared)
    ts = []
    for _ in range(3):
        t0 = time.perf_counter()
        ol.moe_layer_l1_torch(x, ids_n, wt_n, experts, cfg.expert_start, shared)
        ts.append(time.perf_counter() - t0)
    return sorted(ts)[1], threads, n / cfg.n_tokens, \
        f"{n} of {cfg.n_tokens} tokens of the workload, all experts they route to, weights dequantised to bf16 " \
        "beforehand, 1 warm-up + median of 3"


def measure_layer(a, config, with_cpu):
    """One configuration of the layer: K timed passes back to back, K passes with the last-level cache flushed
    before each (decode), K passes with per-launch events for the dominant kernel, and the CPU baseline."""
    import numpy as np
    import torch
    from batchgen_amd import _lib, workloads as wl
    from batchgen_amd.moe.fp8_layer import Fp8MoELayer

    dev = torch.device(DEVICE)
    torch.cuda.set_device(dev)
    cfg = wl.K3_LATENT if config == 5 else wl.CONFIGS[config]
    inp = wl.make_inputs(cfg, dev)
    mx4 = cfg.weight_format == "mxfp4"
    lat = None
    if mx4:
        from batchgen_amd.moe.mxfp4_layer import Mxfp4MoELayer
        w, sh = wl.make_mxfp4_weights(cfg, dev)
        lat = wl.make_latent_weights(cfg, dev) if cfg.latent else None
        kw = {"dense_backend": a.dense_backend} if a.dense_backend else {}
        if getattr(a, "fold_gather", False):
            kw["fold_gather"] = True
        layer = Mxfp4MoELayer(cfg, w, sh, inp["bias"], latent=lat, **kw)
    else:
        w, sh = wl.make_fp8_weights(cfg, dev)
        layer = Fp8MoELayer(cfg, w, sh, inp["bias"])
    _lib.check(_lib.lib().bgmoe_set_tiled_variant(int(getattr(a, "tiled_variant", 0))))
    _lib.check(_lib.lib().bgmoe_set_skinny_tall_min_rows(int(getattr(a, "tall_min_rows", 0))))
    _lib.check(_lib.lib().bgmoe_set_skinny_s1_stages(int(getattr(a, "s1_stages", 3))))
    _lib.check(_lib.lib().bgmoe_set_skinny_gemm_stages(int(getattr(a, "gemm_stages", 2))))
    _lib.check(_lib.lib().bgmoe_set_mxfp4_variant(int(getattr(a, "mxfp4_variant", 0))))
    _lib.check(_lib.lib().bgmoe_set_router_gemm_plan(-1, int(getattr(a, "bf16_gemm_plan", -1))))
    x, logits = inp["x"], inp["logits"]

    for _ in range(a.warmup):
        layer(x, logits)
    torch.cuda.synchronize()
    if a.copy_calibration:
        from batchgen_amd.moe.fp8_layer import repack_tile_major
        cal = torch.zeros((1, 32768, 8192), dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
        repack_tile_major(cal)
        torch.cuda.synchronize()
        del cal
    step = lambda: layer(x, logits)
    if a.graph:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            layer(x, logits)
        step = graph.replay
        step()
        torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(a.steps):
        step()
    stop.record()
    torch.cuda.synchronize()
    ms = start.elapsed_time(stop) / a.steps

    counts = layer.expert_counts[:cfg.e_local].cpu().numpy()
    active = int((counts > 0).sum())
    rows = int(counts.sum())
    alg_bytes = wl.algorithmic_bytes_mxfp4(cfg, active, rows) if mx4 else wl.algorithmic_bytes_fp8(cfg, active, rows)
    flops = wl.flops_routed(cfg, rows) + (cfg.n_tokens * 6 * cfg.hidden * cfg.shared_inter if cfg.shared_inter else 0)
    if cfg.latent:
        flops += cfg.n_tokens * 4 * cfg.hidden * cfg.latent
    decode = cfg.layout == "masked"
    gbps = alg_bytes / (ms * 1e-3) / 1e9
    tflops = flops / (ms * 1e-3) / 1e12

    # the same passes with the last-level cache flushed before each one: a kernel that READS 512 MiB (twice the
    # 256 MiB Infinity Cache; a write would leave dirty lines whose write-back competes with the pass that
    # follows) runs on the stream right before the timed pass, so the pass starts on a busy queue as in the
    # back-to-back loop.  Events bracket the pass only.
    flush = None
    if decode:
        fbuf = torch.zeros(FLUSH_BYTES // 4, dtype=torch.int32, device=dev)
        evs = []
        for _ in range(a.steps):
            fbuf.sum()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            step()
            e1.record()
            evs.append((e0, e1))
        torch.cuda.synchronize()
        fms = float(np.median([e0.elapsed_time(e1) for e0, e1 in evs]))
        del fbuf
        flush = {"bytes_read_before_each_step": FLUSH_BYTES, "ms_per_step": fms,
                 "layer_hbm_GBps": alg_bytes / (fms * 1e-3) / 1e9,
                 "layer_frac_of_hbm_peak": alg_bytes / (fms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                 "note": "median of per-step event times; this is what `value` and ms_per_step report"}

    # second timed pass with per-launch HIP events -> duration of the dominant kernel
    _lib.prof_enable(True)
    for _ in range(a.steps):
        layer(x, logits)
    prof = _lib.prof_collect()
    _lib.prof_enable(False)
    per_kernel = {k: v[0] / a.steps for k, v in prof.items()}          # ms per step
    h, i = cfg.hidden, cfg.inter
    if mx4:
        dom = "mxfp4_s1"
        eh = cfg.expert_hidden
        dom_bytes = active * (2 * eh * i // 2 + 2 * eh * i // 32) + rows * (eh + i) * 2
        dom_ms = prof[dom][0] / max(prof[dom][1], 1)
        roof = dict(bound="hbm", kernel="mxfp4_skinny_kernel<fused,tile_major>",
                    achieved=dom_bytes / (dom_ms * 1e-3) / 1e9, peak=HBM_PEAK_GBPS, unit="GB/s", traffic=None,
                    bytes_per_launch=dom_bytes, avg_launch_us=dom_ms * 1e3)
    elif decode:
        dom = "s1_skinny16"
        # one launch streams gate+up of every active routed expert and of the shared expert once
        # (algorithmic bytes: each weight byte once, each quantised row in, each requantised row out)
        served = active + (1 if cfg.shared_inter else 0)
        srows = rows + (cfg.n_tokens if cfg.shared_inter else 0)
        dom_bytes = served * (2 * h * i + 2 * (h // 128) * (i // 128) * 4) + \
            srows * (h + h // 128 * 4 + i + i // 128 * 4)
        dom_ms = prof[dom][0] / max(prof[dom][1], 1)
        roof = dict(bound="hbm", kernel="fp8_skinny_kernel<fused,tile_major>", achieved=dom_bytes / (dom_ms * 1e-3) / 1e9,
                    peak=HBM_PEAK_GBPS, unit="GB/s", traffic=None, bytes_per_launch=dom_bytes,
                    avg_launch_us=dom_ms * 1e3)
    else:
        dom = "s1_tiled"
        # the device-side rule of the library: groups above 64 rows are tiled when they make >= 8 tiles of 256
        allc = np.append(counts, cfg.n_tokens if cfg.shared_inter else 0)
        lo = 64 if int(((allc[allc > 64] + 255) // 256).sum()) >= 8 else 256
        big = counts[counts > lo].sum()
        dom_flops = int(big) * 4 * h * i + (cfg.n_tokens * 4 * h * cfg.shared_inter if cfg.shared_inter else 0)
        dom_ms = prof[dom][0] / max(prof[dom][1], 1)
        roof = dict(bound="mfma", kernel="fp8_tiled_kernel<fused,tile_major>", achieved=dom_flops / (dom_ms * 1e-3) / 1e12,
                    peak=FP8_PEAK_TFLOPS, unit="TFLOP/s", traffic=None, flops_per_launch=dom_flops,
                    avg_launch_us=dom_ms * 1e3)
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["traffic"], roof["traffic_source"] = traffic_record(f"layer:{config}")
    if not decode and int(getattr(a, "tiled_variant", 0)) != 0:
        roof["kernel"] = "fp8_tiled_k64_kernel<fused,tile_major>"
    if decode and not mx4 and int(getattr(a, "tall_min_rows", 0)) != 0:
        roof["kernel"] = "fp8_skinny_kernel<fused,tile_major,tall items>"

    # Decode: the figure reported as `value` is the cache-flushed one.  A decode step of a real model finds none of
    # this layer's weights in the 256 MiB last-level cache (the other layers' weights have passed through it since),
    # so the back-to-back loop, whose every pass starts with a part of the weights still cached, flatters the layer;
    # it is kept as `back_to_back`.
    b2b = {"ms_per_step": ms, "layer_hbm_GBps": gbps, "layer_frac_of_hbm_peak": gbps / HBM_PEAK_GBPS,
           "tokens_per_s": cfg.n_tokens / (ms * 1e-3),
           "note": "K passes enqueued back to back between two events (no cache flush between passes)"}
    if flush is not None:
        ms = flush["ms_per_step"]
        gbps = alg_bytes / (ms * 1e-3) / 1e9
        tflops = flops / (ms * 1e-3) / 1e12

    out = {
        "metric": METRIC,
        "value": gbps if decode else tflops,
        "unit": "GB/s" if decode else "TFLOP/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": ms,
        "timing": ("median of the K per-step event times, 512 MiB read through the chip before every step "
                   "(last-level cache flushed)") if flush is not None else "K passes back to back between two events",
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "launch": "hip_graph" if a.graph else "eager",
        "dtype": "mxfp4 weights x bf16 (fp32 accumulate)" if mx4 else "fp8_e4m3 (fp32 accumulate)", "data": "synthetic",
        "config": {"workload": cfg.name, "tokens": cfg.n_tokens, "hidden": h, "latent": cfg.latent or None,
                   "activation": cfg.activation, "moe_intermediate": i,
                   "experts": cfg.n_experts, "local_experts": cfg.e_local, "top_k": cfg.top_k,
                   "layout": cfg.layout, "shared_expert": bool(cfg.shared_inter)},
        "tokens_per_s": cfg.n_tokens / (ms * 1e-3),
        "layer_hbm_GBps": gbps, "layer_TFLOPs": tflops,
        "layer_frac_of_hbm_peak": gbps / HBM_PEAK_GBPS, "layer_frac_of_fp8_peak": tflops / FP8_PEAK_TFLOPS,
        "algorithmic_bytes": alg_bytes, "flops": flops, "active_local_experts": active, "routed_rows": rows, "expert_counts": counts.tolist(),
        "kernel_ms_per_step": per_kernel,
        "roofline": roof,
    }
    if flush is not None:
        out["cache_flushed"] = flush
        out["back_to_back"] = b2b
    if getattr(a, "template", False) and not mx4:
        out["template_layer"] = measure_template_layer(a, cfg, inp, w, sh)
    ids = layer.topk_ids.cpu().numpy()
    wt = layer.topk_weights.cpu().numpy()
    if with_cpu and mx4 and cfg.latent:
        t, frac, sample = cpu_baseline_mxfp4(cfg, inp, w, sh, lat)
        out["cpu_baseline"] = {"value": alg_bytes * frac / t / 1e9, "unit": out["unit"],
                               "cores": min(os.cpu_count() or 1, 16), "host_cores": os.cpu_count() or 1,
                               "kind": "port", "sample": sample + " (BLAS threads for the matrix products, one thread for the dequantisation)", "seconds": t,
                               "tokens_per_s": cfg.n_tokens * frac / t}
    elif with_cpu and mx4:
        t, threads, frac, sample = cpu_baseline_mxfp4_torch(cfg, inp, w, sh, ids, wt)
        out["cpu_baseline"] = {"value": alg_bytes * frac / t / 1e9, "unit": out["unit"], "cores": threads,
                               "host_cores": os.cpu_count() or 1, "kind": "port", "sample": sample, "seconds": t,
                               "tokens_per_s": cfg.n_tokens * frac / t}
    elif with_cpu:
        t, threads, cores, sample, frac = cpu_baseline(cfg, inp, w, sh, ids, wt, alg_bytes, flops)
        v = (alg_bytes * frac / t / 1e9) if decode else (flops * frac / t / 1e12)
        out["cpu_baseline"] = {"value": v, "unit": out["unit"], "cores": threads, "host_cores": cores,
                               "kind": "port", "sample": sample, "seconds": t,
                               "tokens_per_s": cfg.n_tokens * frac / t}
    del layer, w, sh, inp, x, logits
    torch.cuda.empty_cache()
    return out


def measure_template_layer(a, cfg, inp, w, sh):
    """The same weights behind the reference's layer template (batchgen_amd.moe.moe_base.Fp8BlockwiseMoE built from a
    model configuration object): router GEMM + gate as one op, the routed experts behind the routes it returns, the
    dense FP8 shared expert, the add -- what a model file's decode path runs, timed like the one-call layer."""
    from types import SimpleNamespace
    import torch
    from batchgen_amd.moe.moe_base import Fp8BlockwiseMoE
    dev = inp["x"].device
    mc = SimpleNamespace(hidden_size=cfg.hidden, moe_intermediate_size=cfg.inter, n_routed_experts=cfg.n_experts,
                         num_experts_per_tok=cfg.top_k, n_group=cfg.n_group, topk_group=cfg.topk_group,
                         routed_scaling_factor=cfg.rsf, norm_topk_prob=True,
                         n_shared_experts=1 if cfg.shared_inter else 0,
                         phase="decode" if cfg.layout == "masked" else "prefill")
    g = torch.Generator(device="cpu").manual_seed(4242)
    gate_w = (torch.randn(cfg.n_experts, cfg.hidden, generator=g) * 0.05).to(torch.bfloat16).to(dev)
    bias = (torch.randn(cfg.n_experts, generator=g) * 0.1).to(dev)
    layer = Fp8BlockwiseMoE(mc, w, sh if cfg.shared_inter else None, gate_w, bias)
    # one process stands for the rank that holds this share: the gate routes over all experts, the local range is
    # the configuration's (the template derives it from the world size, which is 1 here)
    layer.experts_per_rank = layer.num_persistent_local_experts = cfg.e_local
    layer.routed_expert_start_idx, layer.routed_expert_end_idx = cfg.expert_start, cfg.expert_start + cfg.e_local
    layer.set_num_tokens_per_rank(cfg.n_tokens)
    x = inp["x"]
    for _ in range(a.warmup):
        layer(x)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(a.steps):
        layer(x)
    stop.record()
    torch.cuda.synchronize()
    ms = start.elapsed_time(stop) / a.steps
    return {"ms_per_step": ms, "tokens_per_s": cfg.n_tokens / (ms * 1e-3), "launch": "eager",
            "routed_rows": int(layer._routed.expert_counts[:cfg.e_local].sum()),
            "note": "router GEMM + gate on the hidden states with a random gate weight (the one-call layer is given "
                    "logits), routed experts of the same local range behind the returned routes, dense shared "
                    "expert, add: the launches of a model file's decode path"}


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py measures one GPU's expert-parallel share; this build has no multi-GPU path "
              "(run with --gpus 1).", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    if a.op != "layer":
        return bench_producer(a)
    if a.config is not None:
        print(json.dumps(measure_layer(a, a.config, not a.no_cpu_baseline)))
        return
    # Default run: the metric has two halves.  The line is configuration 1 (decode: HBM GB/s, the figure `value`
    # reports); its "prefill" object is configuration 2 (prefill: FP8 TFLOP/s) measured the same way in the same
    # process, with fewer steps because one prefill pass is ten times longer.
    out = measure_layer(a, 1, not a.no_cpu_baseline)
    import copy
    b = copy.copy(a)
    b.steps, b.warmup = max(5, a.steps // 4), max(2, a.warmup // 2)
    pre = measure_layer(b, 2, not a.no_cpu_baseline)
    keep = ("value", "unit", "steps", "warmup", "ms_per_step", "launch", "dtype", "config", "tokens_per_s", "layer_TFLOPs",
            "layer_frac_of_fp8_peak", "flops", "active_local_experts", "routed_rows", "kernel_ms_per_step", "roofline",
            "cpu_baseline")
    out["prefill"] = {k: pre[k] for k in keep if k in pre}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
