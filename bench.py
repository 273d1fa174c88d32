#!/usr/bin/env python3
"""Benchmark of the hot path: 4-bit block GEMV at Llama-3-8B layer shapes.

One step = the projection GEMVs of one decode token: for each of 32 decoder
layers (distinct weights, 3.9 GB packed in total, so nothing is served from
cache) q 4096x4096, k/v 1024x4096, o 4096x4096, gate/up 14336x4096 and down
4096x14336, batch 1, bf16 activations, fp32 outputs.  Inputs are the seeded
streams of the reference's generator (quant::RNG, src/core/random.cpp:45-81,
through the library's own RNG mirror): weights RNG(42).normal() * 0.02 for one
decoder layer, rotated by a different offset for every further layer, quantized
on the device to the 4-bit block-32 binary16-scale format (B32S4, 4.5 bits per
weight); activations RNG(43).normal() rounded to bf16; Laplace weights from
RNG(44); router logits from RNG(45).  Everything is resident in HBM before
timing starts.

Prints one JSON line.  value = algorithmic bytes per step / wall time per step.
"""
from __future__ import annotations

import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes moved per algorithmic byte for the GEMV launches of this workload, from
# rocprofv3 FETCH_SIZE / WRITE_SIZE scaled by a 1 GiB copy kernel (summary under profiles/)
HBM_TRAFFIC_RATIO = 1.0245
# (name, N, K, input) per decoder layer
PROJ = [("q", 4096, 4096, "x"), ("k", 1024, 4096, "x"), ("v", 1024, 4096, "x"), ("o", 4096, 4096, "a"),
        ("gate", 14336, 4096, "x"), ("up", 14336, 4096, "x"), ("down", 4096, 14336, "h")]


def alg_bytes(N, K, B, bpw, sx=2, sy=4):
    return N * K * bpw / 8 + B * K * sx + B * N * sy


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--fmt", default="B32S4")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-prefill", action="store_true", help="skip the prefill GEMM figure")
    ap.add_argument("--no-moe", action="store_true", help="skip the mixture-of-experts layer figure")
    ap.add_argument("--no-chain", action="store_true",
                    help="skip the figure of the same step as one persistent launch (tfq_chain_*: true data dependencies)")
    ap.add_argument("--no-sweep", action="store_true",
                    help="skip the batch / format sweep (batch 4, 8, 16; the 8-bit format; the low-bit superblock formats)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one elementwise kernel that reads and writes 1 GiB (counter calibration)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus above 1 is not supported "
              "(rows of a matrix would shard over GPUs without a collective; that is not built)", file=sys.stderr)
        sys.exit(2)

    import torch
    tfq = importlib.import_module("transformers-fusion_amd")
    tfq.init(0)
    dev = torch.device("cuda:0")
    B, fmt = args.batch, args.fmt
    bpw = float(tfq.lib().tfq_format_bpw(tfq.fmt_id(fmt)))

    # one decoder layer from RNG(42), the projections in PROJ order on one stream
    total = sum(N * K for _, N, K, _ in PROJ)
    w_all = torch.from_numpy(tfq.rng_normal(42, total, 0.02)).to(dev)
    base, at = {}, 0
    for name, N, K, _ in PROJ:
        base[name] = w_all[at:at + N * K]
        at += N * K
    layers, host_layer0 = [], {}
    for li in range(args.layers):
        ws = {}
        for name, N, K, _ in PROJ:
            w = base[name] if li == 0 else torch.roll(base[name], li * 1000003)
            packed = tfq.encode(fmt, w)
            ws[name] = tfq.Weight(fmt, N, K, packed)
            if li == 0 and not args.no_cpu:
                host_layer0[name] = packed.cpu().numpy()  # wire payload for the CPU baseline
            del w, packed
        layers.append(ws)
    a_all = torch.from_numpy(tfq.rng_normal(43, B * (4096 + 4096 + 14336))).to(dev)
    acts = {"x": a_all[:B * 4096].reshape(B, 4096).bfloat16(),
            "a": a_all[B * 4096:2 * B * 4096].reshape(B, 4096).bfloat16(),
            "h": a_all[2 * B * 4096:].reshape(B, 14336).bfloat16()}
    outs = {name: torch.empty(B, N, device=dev, dtype=torch.float32) for name, N, _, _ in PROJ}
    torch.cuda.synchronize()

    # launches per layer follow the data dependencies of a decoder layer: q/k/v share the
    # layer input and go in one launch, so do gate/up; o and down are launches of their own
    def step():
        for ws in layers:
            tfq.gemv_multi([ws["q"], ws["k"], ws["v"]], acts["x"], [outs["q"], outs["k"], outs["v"]])
            ws["o"].gemv(acts["a"], out=outs["o"])
            tfq.gemv_multi([ws["gate"], ws["up"]], acts["x"], [outs["gate"], outs["up"]])
            ws["down"].gemv(acts["h"], out=outs["down"])

    launches_per_step = args.layers * 4
    bytes_per_step = args.layers * sum(alg_bytes(N, K, B, bpw) for _, N, K, _ in PROJ)

    if args.calibrate_copy:  # known traffic for scaling FETCH_SIZE / WRITE_SIZE readings
        src = torch.zeros(1 << 28, device=dev, dtype=torch.float32)
        dst = torch.empty_like(src)
        torch.add(src, 1.0, out=dst)
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    graph = None
    if not args.no_graph:
        try:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                step()
            graph.replay()
            torch.cuda.synchronize()
        except Exception as e:  # plain launches still measure the same kernels
            print(f"[bench] graph capture unavailable ({e}); timing plain launches", file=sys.stderr)
            graph = None
    run = graph.replay if graph is not None else step

    # timed region: exactly K steps, wall clock for `value`, HIP events on the
    # launch stream for the kernel-side duration
    stream = torch.cuda.current_stream()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record(stream)
    for _ in range(args.steps):
        run()
    e1.record(stream)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    ev_ms_per_step = e0.elapsed_time(e1) / args.steps

    value = bytes_per_step / (ms_per_step * 1e-3) / 1e9
    avg_launch_us = ev_ms_per_step * 1e3 / launches_per_step
    achieved = (bytes_per_step / launches_per_step) / (avg_launch_us * 1e-6) / 1e9

    res = {
        "metric": "4-bit block GEMV achieved HBM GB/s, Llama-3-8B layer shapes, batch %d" % B,
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic: quant::RNG streams (seed 42 weights N(0, 0.02), one layer, rotated per layer; seed 43 "
                "activations N(0, 1) as bf16; 44 Laplace; 45 router logits)",
        "config": {"workload": "llama3-8b decode projections (q,k,v,o,gate,up,down) x %d layers, batch %d, "
                               "%s weights, bf16 activations, fp32 outputs" % (args.layers, B, fmt),
                   "format": fmt, "layers": args.layers, "batch": B, "launch": "hipGraph" if graph else "stream"},
        "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
        "decode_tok_s": round(1e3 / (ms_per_step * 32.0 / args.layers), 1),
        "bytes_per_step": int(bytes_per_step),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": int(bytes_per_step / launches_per_step * HBM_TRAFFIC_RATIO),
                     "kernel": "gemv4_kernel", "avg_launch_us": round(avg_launch_us, 3),
                     "alg_bytes_per_launch": int(bytes_per_step / launches_per_step)},
    }

    if not args.no_chain and B <= 2 and fmt in ("B32S4", "Q_G_4"):
        res["chain"] = chain_step(tfq, torch, layers, bytes_per_step)
        res["fused_launches"] = fused_launch_step(tfq, torch, layers, bytes_per_step)
    if not args.no_prefill:
        res["prefill"] = prefill_gemm(tfq, torch, layers[0])
    if not args.no_sweep:
        res["sweep"] = decode_sweep(tfq, torch, layers, fmt, base)
    if not args.no_moe:
        del layers
        torch.cuda.empty_cache()
        res["moe"] = moe_layer(tfq, torch, fmt, bpw, base)
    if not args.no_sweep:
        res["output_projection"] = output_projection(tfq, torch, fmt, bpw, base)
    if not args.no_cpu:
        # the reference caps its matmul at 8 threads (src/adapters/tools/qwen35_engine.cpp:60); the second
        # figure uses every core this process may use
        res["cpu_baseline"] = cpu_baseline(host_layer0, fmt, B, acts, bpw, threads=min(8, usable_cores()))
        res["cpu_baseline_all_cores"] = cpu_baseline(host_layer0, fmt, B, acts, bpw, threads=usable_cores(), budget_s=8.0)
    print(json.dumps(res), flush=True)


def chain_step(tfq, torch, layers, bytes_per_step, reps=20):
    """The same projections as ONE persistent launch with the data dependencies of a decoder layer kept inside
    the kernel (rmsnorm -> q, k, v | o(q) -> h += . | rmsnorm -> gate, up -> silu * up -> down -> h += ., attention
    itself is outside the path, so o takes q): a side figure, never `value`."""
    dev = "cuda"
    h = torch.from_numpy(tfq.rng_normal(43, 4096)).to(dev).reshape(1, 4096)
    gamma = torch.zeros(4096, device=dev)
    phases = []
    for li, ws in enumerate(layers):
        phases += [
            {"w": [ws["q"], ws["k"], ws["v"]], "x": h if li == 0 else None, "x_op": tfq.X_RMSNORM, "gamma": gamma, "gamma_plus_one": True},
            {"w": [ws["o"]], "y_op": tfq.Y_RESIDUAL, "residual": h},
            {"w": [ws["gate"], ws["up"]], "x_op": tfq.X_RMSNORM, "gamma": gamma, "gamma_plus_one": True, "y_op": tfq.Y_SWIGLU},
            {"w": [ws["down"]], "y_op": tfq.Y_RESIDUAL, "residual": h},
        ]
    if len(phases) > 128:
        return {"skipped": "more than 128 phases"}
    chain = tfq.Chain(phases, B=1)
    h_start = h.clone()
    chain.run()
    torch.cuda.synchronize()
    chain.check()
    # the hidden state after one step against the same sequence as fused launches from the same start (the chain hands
    # q on to o as bf16, the launches as fp32, so the two agree to bf16 rounding carried through 32 layers: 1-2 %)
    h_chain = h.clone()
    href = h_start.clone()
    q, k, v = (torch.empty(1, n, device=dev) for n in (4096, 1024, 1024))
    mid = torch.empty(1, 14336, device=dev, dtype=torch.bfloat16)
    for ws in layers:
        tfq.gemv_multi_fused([ws["q"], ws["k"], ws["v"]], href, [q, k, v], rmsnorm=gamma)
        tfq.gemv_multi_fused([ws["o"]], q, [href], accumulate=True)
        tfq.gemv_multi_fused([ws["gate"], ws["up"]], href, [mid], rmsnorm=gamma, pair_swiglu=True)
        tfq.gemv_multi_fused([ws["down"]], mid, [href], accumulate=True)
    torch.cuda.synchronize()
    diff = float((h_chain - href).abs().max() / href.abs().max())
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        chain.run()
    e1.record()
    torch.cuda.synchronize()
    chain.check()
    us = e0.elapsed_time(e1) * 1e3 / reps
    chain.close()
    return {"launches_per_step": 1, "phases": len(phases), "us_per_step": round(us, 1), "us_per_layer": round(us / len(layers), 2),
            "gbs": round(bytes_per_step / us / 1e3, 1), "frac": round(bytes_per_step / us / 1e3 / HBM_PEAK_GBS, 4),
            "max_diff_vs_fused_launches": diff,
            "note": "dependent phases inside one launch, RMSNorm / SwiGLU / residual fused"}


def fused_launch_step(tfq, torch, layers, bytes_per_step):
    """The same dependent decoder-layer sequence as four launches per layer with every elementwise step inside the
    launches (tfq_gemv_multi_fused: RMSNorm in front of q/k/v and gate/up, SwiGLU in the epilogue of the paired
    gate/up launch, the residual additions in the epilogues of o and down), fp32 hidden state, bf16 SwiGLU product.
    A side figure, never `value`."""
    dev = "cuda"
    h = torch.from_numpy(tfq.rng_normal(43, 4096)).to(dev).reshape(1, 4096)
    gamma = torch.zeros(4096, device=dev)
    q, k, v = (torch.empty(1, n, device=dev) for n in (4096, 1024, 1024))
    mid = torch.empty(1, 14336, device=dev, dtype=torch.bfloat16)

    def step():
        for ws in layers:
            tfq.gemv_multi_fused([ws["q"], ws["k"], ws["v"]], h, [q, k, v], rmsnorm=gamma)
            tfq.gemv_multi_fused([ws["o"]], q, [h], accumulate=True)
            tfq.gemv_multi_fused([ws["gate"], ws["up"]], h, [mid], rmsnorm=gamma, pair_swiglu=True)
            tfq.gemv_multi_fused([ws["down"]], mid, [h], accumulate=True)
    us = time_graph(torch, step)
    return {"launches_per_layer": 4, "us_per_layer": round(us / len(layers), 2), "gbs": round(bytes_per_step / us / 1e3, 1),
            "frac": round(bytes_per_step / us / 1e3 / HBM_PEAK_GBS, 4),
            "note": "fp32 hidden state; RMSNorm, SwiGLU and the residual additions fused into the 4 GEMV launches of a layer"}


def time_graph(torch, fn, reps=10):
    """us per call of fn (launches on the current stream), from graph replays when capture works."""
    fn()
    torch.cuda.synchronize()
    run = fn
    try:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            fn()
        g.replay()
        run = g.replay
    except Exception:
        pass
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        run()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / reps


def decode_sweep(tfq, torch, layers, fmt, base):
    """Side figures, never `value`: the decode layer of the main workload at batch 4, 8 and 16 (same weights,
    same four launches per layer), the 8-bit block-32 format at batch 1, 4, 8 and 16 on eight layers, and the low-bit
    superblock formats (Laplace(0, 0.015) weights, 14336x4096, twelve rotated copies) at batch 1 and 8.
    GB/s = algorithmic bytes / time, as for `value`."""
    dev = "cuda"
    out = {}

    def layer_step(ls, B):
        a_all = torch.from_numpy(tfq.rng_normal(43, B * (4096 + 4096 + 14336))).to(dev)
        acts = {"x": a_all[:B * 4096].reshape(B, 4096).bfloat16(), "a": a_all[B * 4096:2 * B * 4096].reshape(B, 4096).bfloat16(),
                "h": a_all[2 * B * 4096:].reshape(B, 14336).bfloat16()}
        outs = {name: torch.empty(B, N, device=dev, dtype=torch.float32) for name, N, _, _ in PROJ}

        def step():
            for ws in ls:
                tfq.gemv_multi([ws["q"], ws["k"], ws["v"]], acts["x"], [outs["q"], outs["k"], outs["v"]])
                ws["o"].gemv(acts["a"], out=outs["o"])
                tfq.gemv_multi([ws["gate"], ws["up"]], acts["x"], [outs["gate"], outs["up"]])
                ws["down"].gemv(acts["h"], out=outs["down"])
        return step

    def layer_figures(ls, f, B):
        bpw = float(tfq.lib().tfq_format_bpw(tfq.fmt_id(f)))
        us = time_graph(torch, layer_step(ls, B)) / len(ls)
        nbytes = sum(alg_bytes(N, K, B, bpw) for _, N, K, _ in PROJ)
        return {"us_per_layer": round(us, 2), "gbs": round(nbytes / us / 1e3, 1),
                "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4), "tok_s": round(B * 1e6 / (us * 32.0), 1)}

    out[fmt] = {str(B): layer_figures(layers, fmt, B) for B in (4, 8, 16)}
    ls8 = []
    for li in range(8):
        ws = {}
        for name, N, K, _ in PROJ:
            w = base[name] if li == 0 else torch.roll(base[name], li * 1000003)
            ws[name] = tfq.Weight("B32S8", N, K, tfq.encode("B32S8", w))
            del w
        ls8.append(ws)
    out["B32S8"] = {str(B): layer_figures(ls8, "B32S8", B) for B in (1, 4, 8, 16)}
    for ws in ls8:
        for W in ws.values():
            W.close()
    del ls8
    N, K = 14336, 4096
    u = torch.from_numpy(tfq.rng_uniform(44, N * K)).to(dev) - 0.5
    lap = -0.015 * torch.sign(u) * torch.log1p(-2.0 * u.abs())  # Laplace(0, 0.015) by inverse CDF
    del u
    for f in ("SB256A3", "SB256A2"):
        bpw = float(tfq.lib().tfq_format_bpw(tfq.fmt_id(f)))
        Ws = []
        for c in range(12):
            w = lap if c == 0 else torch.roll(lap, c * 1000003)
            Ws.append(tfq.Weight(f, N, K, tfq.encode(f, w)))
            del w
        out[f] = {}
        for B in (1, 8):
            x = torch.from_numpy(tfq.rng_normal(43, B * K)).to(dev).reshape(B, K).bfloat16()
            y = torch.empty(B, N, device=dev, dtype=torch.float32)

            def step():
                for W in Ws:
                    W.gemv(x, out=y)
            us = time_graph(torch, step) / len(Ws)
            nbytes = alg_bytes(N, K, B, bpw)
            out[f][str(B)] = {"shape": "%dx%d" % (N, K), "us": round(us, 2), "gbs": round(nbytes / us / 1e3, 1),
                              "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)}
        for W in Ws:
            W.close()
        del Ws
    return out


MFMA_PEAK_TFLOPS = 2500.0


def prefill_gemm(tfq, torch, layer, M=2048, reps=10):
    """The prefill GEMM on the same weights: M = 2048 bf16 tokens through gate (14336x4096) and down
    (4096x14336), bf16 output, fp32 accumulation on the matrix cores.  A side figure, not `value`."""
    out = {"tokens": M, "peak_tflops": MFMA_PEAK_TFLOPS, "bound": "mfma"}
    for name in ("gate", "down"):
        W = layer[name]
        x = torch.from_numpy(tfq.rng_normal(43, M * W.K)).to("cuda").reshape(M, W.K).bfloat16()
        for _ in range(3):
            y = W.gemm(x, out_dtype=torch.bfloat16)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            y = W.gemm(x, out_dtype=torch.bfloat16)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        tf = 2.0 * M * W.N * W.K / (ms * 1e-3) / 1e12
        out[name] = {"shape": "%dx%d" % (W.N, W.K), "us": round(ms * 1e3, 1), "tflops": round(tf, 1),
                     "frac": round(tf / MFMA_PEAK_TFLOPS, 4)}
        # For scale, on the same box (they differ by up to 20 % on this shape): the vendor library's plain
        # bf16 GEMM (torch.matmul) on the same matrix decoded to bf16 beforehand, i.e. with no decode in the
        # loop and four times the weight bytes.  A comparator only: nothing in the library calls it.
        wd = W.decode().bfloat16()
        yl = torch.empty((M, W.N), dtype=torch.bfloat16, device="cuda")
        for _ in range(3):
            torch.matmul(x, wd.T, out=yl)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(reps):
            torch.matmul(x, wd.T, out=yl)
        e1.record()
        torch.cuda.synchronize()
        ms_lib = e0.elapsed_time(e1) / reps
        out[name]["library_bf16_gemm_us"] = round(ms_lib * 1e3, 1)
        out[name]["library_bf16_gemm_tflops"] = round(2.0 * M * W.N * W.K / (ms_lib * 1e-3) / 1e12, 1)
        out[name]["max_diff_vs_library"] = float((y.float() - yl.float()).abs().max() / yl.float().abs().max())
        del x, y, wd, yl
    return out


def moe_layer(tfq, torch, fmt, bpw, base, E=8, top_k=2, T=16, D=4096, F=14336, reps=20):
    """One mixture-of-experts FFN call (router top-k given on the host, like the reference's dispatch):
    16 tokens, 8 experts, top-2, gate/up 14336x4096 and down 4096x14336 per expert.  Wall time per call
    including the host-side routing lists; bytes = packed weights of the active experts.  A side figure."""
    import numpy as np
    gate, up, down = [], [], []
    for e in range(E):  # expert e = the layer's gate / up / down stream rotated by e * 1000003 elements
        for lst, name, n, k in ((gate, "gate", F, D), (up, "up", F, D), (down, "down", D, F)):
            w = base[name] if e == 0 else torch.roll(base[name], e * 1000003)
            lst.append(tfq.Weight(fmt, n, k, tfq.encode(fmt, w)))
            del w
    logits = torch.from_numpy(tfq.rng_normal(45, T * E)).to("cuda").reshape(T, E)
    _, idx, wts = tfq.moe_route(logits, top_k)
    idx_h, w_h = idx.cpu().numpy().astype(np.int64), wts.cpu().numpy()
    x = torch.from_numpy(tfq.rng_normal(43, T * D)).to("cuda").reshape(T, D).bfloat16()
    for _ in range(3):
        tfq.moe_ffn(gate, up, down, idx_h, w_h, x, mid_dtype=torch.bfloat16)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        tfq.moe_ffn(gate, up, down, idx_h, w_h, x, mid_dtype=torch.bfloat16)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / reps
    active = len(set(idx_h.reshape(-1).tolist()))
    nbytes = active * 3 * F * D * bpw / 8
    out = {"tokens": T, "experts": E, "top_k": top_k, "active_experts": active,
           "tokens_per_expert": [int((idx_h == e).sum()) for e in range(E)],
           "us_per_call": round(dt * 1e6, 1), "gbs": round(nbytes / dt / 1e9, 1),
           "frac": round(nbytes / dt / 1e9 / HBM_PEAK_GBS, 4), "bound": "hbm"}
    # the same call with the routing arrays left on the device (lists and launch tables built there), as graph replays
    routed = tfq.RoutedMoe(gate, up, down, T, top_k)
    y = torch.empty(T, D, device="cuda")
    for _ in range(3):
        routed(idx, wts, x, y)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        routed(idx, wts, x, y)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        routed(idx, wts, x, y)
    for _ in range(3):
        g.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        g.replay()
    torch.cuda.synchronize()
    dtr = (time.perf_counter() - t0) / reps
    out["routed_on_device"] = {"us_per_call": round(dtr * 1e6, 1), "gbs": round(nbytes / dtr / 1e9, 1),
                               "frac": round(nbytes / dtr / 1e9 / HBM_PEAK_GBS, 4),
                               "note": "routing arrays on the device, lists built there, graph replays"}
    # one token (the decode step of a single sequence): two active experts, the same entry point
    routed1 = tfq.RoutedMoe(gate, up, down, 1, top_k)
    _, idx1, wts1 = tfq.moe_route(logits[:1].contiguous(), top_k)
    x1, y1 = x[:1].contiguous(), torch.empty(1, D, device="cuda")
    for _ in range(3):
        routed1(idx1, wts1, x1, y1)
    torch.cuda.synchronize()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        routed1(idx1, wts1, x1, y1)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g1 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g1):
        routed1(idx1, wts1, x1, y1)
    for _ in range(3):
        g1.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        g1.replay()
    torch.cuda.synchronize()
    dt1 = (time.perf_counter() - t0) / reps
    active1 = len(set(idx1.cpu().numpy().reshape(-1).tolist()))
    nbytes1 = active1 * 3 * F * D * bpw / 8
    out["single_token"] = {"active_experts": active1, "us_per_call": round(dt1 * 1e6, 1), "gbs": round(nbytes1 / dt1 / 1e9, 1),
                           "frac": round(nbytes1 / dt1 / 1e9 / HBM_PEAK_GBS, 4)}
    return out


def output_projection(tfq, torch, fmt, bpw, base, N=128256, K=4096, copies=3, reps=10):
    """The model's largest single GEMV, the projection onto its vocabulary (128256 x 4096, 295 MB packed), at batch
    1 and 8: three copies cut from the layer's weight stream at different offsets, called in rotation (885 MB, more
    than the caches hold), in graph replays.  A side figure: a decode step runs it once per token, `value` covers
    the decoder layers only."""
    stream = torch.cat([base[n] for n in ("gate", "up", "down", "q", "o", "k", "v")])
    need = N * K
    reps_of_stream = (need + (copies - 1) * 1000003) // stream.numel() + 1
    big = stream.repeat(reps_of_stream)
    Ws = [tfq.Weight(fmt, N, K, tfq.encode(fmt, big[i * 1000003:i * 1000003 + need])) for i in range(copies)]
    del big, stream
    out = {"shape": "%dx%d" % (N, K), "packed_mb": round(N * K * bpw / 8 / 1e6, 1)}
    for B in (1, 8):
        x = torch.from_numpy(tfq.rng_normal(43, B * K)).to("cuda").reshape(B, K).bfloat16()
        y = torch.empty(B, N, device="cuda")
        for W in Ws:
            W.gemv(x, out=y)
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            Ws[0].gemv(x, out=y)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        rounds = 8  # launches per replay: 24, so that the replay's own start-up does not weigh on a launch
        with torch.cuda.graph(g):
            for _ in range(rounds):
                for W in Ws:
                    W.gemv(x, out=y)
        for _ in range(2):
            g.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            g.replay()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / (reps * copies * rounds)
        nbytes = N * K * bpw / 8 + B * K * 2 + B * N * 4
        out[str(B)] = {"us": round(dt * 1e6, 2), "gbs": round(nbytes / dt / 1e9, 1), "frac": round(nbytes / dt / 1e9 / HBM_PEAK_GBS, 4)}
    for W in Ws:
        W.close()
    return out


def usable_cores():
    """Cores this process may run on (the scheduler affinity), at most 16: a one-GPU box gives a job that share."""
    try:
        n = len(os.sched_getaffinity(0))
    except AttributeError:
        n = os.cpu_count() or 1
    return max(1, min(16, n))


def cpu_baseline(layer, fmt, B, acts, bpw, threads, budget_s=12.0):
    """The oracle's block-row matmul (reference loop structure: rows split over threads,
    decode 256 weights, 256-long fp32 dot per activation row) on the host cores, on a
    bounded sample: the seven projections of ONE decoder layer, repeated until about
    `budget_s` seconds of CPU work have been timed, on `threads` threads."""
    import oracle as O
    xs = {k: v.float().cpu().numpy() for k, v in acts.items()}
    total_b, total_t, passes = 0.0, 0.0, 0
    while total_t < budget_s and passes < 400:
        for name, N, K, src in PROJ:
            t0 = time.perf_counter()
            O.matmul(fmt, layer[name], N, K, xs[src], threads=threads)
            total_t += time.perf_counter() - t0
            total_b += alg_bytes(N, K, B, bpw)
        passes += 1
    return {"value": round(total_b / total_t / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": "the 7 projections of one decoder layer (%.1f MB packed), %d passes, %.1f s of CPU time"
                      % (sum(alg_bytes(N, K, B, bpw) for _, N, K, _ in PROJ) / 1e6, passes, total_t)}


if __name__ == "__main__":
    main()
