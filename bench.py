#!/usr/bin/env python3
"""Benchmark of the decode-step hot path on one MI355X.

A step is one decoded token: embedding row -> all decoder layers (RMSNorm, QKV/O/FFN GEMVs over f16 weights,
RoPE, f32->f16 KV append, last-token GQA attention over the f16 KV cache) -> output norm -> lm_head GEMV ->
greedy sample.  Workload at N=1: the TinyLlama-1.1B-shaped random-init model of BASELINE.json configs[1]
(22 layers, hidden 2048, 32/4 heads, head_dim 64, FFN 5632, vocab 32000, f16 weights N(0,0.02)), 32 random prompt
ids, then greedy decode at batch 1.  Weights and KV cache are resident in HBM before the timed region.

Prints ONE JSON line: value = decoded tokens per second (whole job); roofline = the dominant kernel's algorithmic
bytes per launch over its event-timed launch duration against 8 TB/s, plus its measured HBM traffic and the time of a
kernel that only reads the same number of bytes in one launch (the practical ceiling on this box); cpu_baseline =
the CPU oracle timed on this host on a short sample of the same workload.  config.b8 carries the batch-8 half of the
metric (Qwen2.5-3B-shaped model, 8 rows), measured in the same run.
"""
import argparse
import ctypes as C
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0     # MI355X HBM3E, published


def algorithmic_bytes_per_token(cfg):
    """Minimum HBM traffic of one decoded token at batch 1: every layer weight and the lm_head once (f16)."""
    D, F, V, L = cfg["d_model"], cfg["ffn"], cfg["vocab"], cfg["n_layers"]
    KV = cfg["kv_heads"] * cfg["head_dim"]
    per_layer = (D * D * 2 + 2 * KV * D + 3 * F * D) * 2
    return L * per_layer + V * D * 2


def chain_cost_us(ctx, n_layers, before, kernel, after, reps=3):
    """What a kernel costs inside the chain of launches it runs in: the chain before(l), kernel(l), after(l) over all
    layers between one pair of events on the decode stream, minus the same chain without the kernel, per layer.  Unlike
    an event pair around every single launch this puts nothing between the launches, and unlike launches of one kernel
    back to back it keeps the dependency on the launch before and the ramp that follows from it."""
    e0, e1 = ctx.event(), ctx.event()

    def run(with_kernel):
        best = None
        for rep in range(reps + 1):          # the first pass warms up
            ctx.sync(1)
            ctx.record(e0, 1)
            for l in range(n_layers):
                before(l)
                if with_kernel:
                    kernel(l)
                after(l)
            ctx.record(e1, 1)
            ms = ctx.elapsed_ms(e0, e1)
            if rep > 0 and (best is None or ms < best):
                best = ms
        return best
    full, rest = run(True), run(False)
    ctx.event_destroy(e0); ctx.event_destroy(e1)
    return (full - rest) * 1e3 / n_layers


def measure_dominant_kernel(pkg, ctx, dm, cfg, reps, mode):
    """Average launch duration of the kernel that moves most of the bytes of a token, timed with HIP events on
    the library's decode stream.  Fused modes: RMSNorm + FFN gate/up GEMV + SwiGLU in one launch (two f16 GGUF
    matrices of N=ffn, K=hidden).  Reference call sequence: the gate (or up) GEMV alone.  Launches cycle through
    the layers' own weight matrices so that no launch finds its weights in a cache."""
    D, F, L = cfg["d_model"], cfg["ffn"], cfg["n_layers"]
    x = ctx.to_device(np.random.default_rng(1).standard_normal(D).astype(np.float32))
    y = ctx.alloc(F * 4)
    lib = ctx.lib
    if mode >= 1:
        def launch(l):
            ly = dm.layers[l]
            return lib.m40llm_ext_fused_norm_gate_up_swiglu_async(ctx.h, x.ptr, ly.ffn_norm, 1, cfg["rms_eps"], ly.wgate,
                                                                  ly.wup, y.ptr, F, D)
        n_variants = L
        name, shape = "norm_gate_up_swiglu_kernel", f"M=1 N=2x{F} K={D}"
        bytes_per_launch = 2 * F * D * 2 + 2 * D * 4 + F * 4      # two matrices + x + norm weights in, hidden out
    else:
        mats = []
        for l in range(L):
            mats.append(dm.layers[l].wgate); mats.append(dm.layers[l].wup)

        def launch(i):
            return lib.m40llm_ext_gemm_f32xf16_gguf_f32_async(ctx.h, x.ptr, mats[i], y.ptr, 1, F, D, 1)
        n_variants = len(mats)
        name, shape = "gemv_f32xf16_gguf_kernel", f"M=1 N={F} K={D}"
        bytes_per_launch = F * D * 2 + D * 4 + F * 4              # weights + activations in + out
    for i in range(n_variants):      # warm-up: code objects, clocks
        pkg.check(launch(i), name)
    ctx.sync(1)
    e0, e1 = ctx.event(), ctx.event()
    ctx.record(e0, 1)
    n = 0
    for r in range(reps):
        for i in range(n_variants):
            launch(i)
            n += 1
    ctx.record(e1, 1)
    ms = ctx.elapsed_ms(e0, e1)
    ctx.event_destroy(e0); ctx.event_destroy(e1)
    out = dict(kernel=name, shape=shape, launches=n, avg_us=ms * 1e3 / n, bytes=bytes_per_launch, in_token_us=None,
               in_chain_us=None)
    if mode >= 1:
        # The same kernel as it runs inside a token: behind the O-projection launch it depends on and before the down
        # projection, one event pair per launch (back-to-back launches of one kernel overlap their ramps; these do not).
        h = ctx.alloc(D * 4); x1 = ctx.alloc(D * 4)
        pairs = [(ctx.event(), ctx.event()) for _ in range(L)]
        for rep in range(2):                      # the first pass warms up
            for l in range(L):
                ly = dm.layers[l]
                lib.m40llm_ext_gemv_residual_f32xf16_async(ctx.h, x.ptr, ly.wo, x.ptr, x1.ptr, D, D)
                ctx.record(pairs[l][0], 1)
                lib.m40llm_ext_fused_norm_gate_up_swiglu_async(ctx.h, x1.ptr, ly.ffn_norm, 1, cfg["rms_eps"], ly.wgate, ly.wup,
                                                               y.ptr, F, D)
                ctx.record(pairs[l][1], 1)
                lib.m40llm_ext_gemv_residual_f32xf16_async(ctx.h, y.ptr, ly.wdown, x1.ptr, h.ptr, D, F)
            ctx.sync(1)
        out["in_token_us"] = sum(ctx.elapsed_ms(a, b) for a, b in pairs) * 1e3 / L
        for a, b in pairs:
            ctx.event_destroy(a); ctx.event_destroy(b)
        out["in_chain_us"] = chain_cost_us(
            ctx, L,
            lambda l: lib.m40llm_ext_gemv_residual_f32xf16_async(ctx.h, x.ptr, dm.layers[l].wo, x.ptr, x1.ptr, D, D),
            lambda l: lib.m40llm_ext_fused_norm_gate_up_swiglu_async(ctx.h, x1.ptr, dm.layers[l].ffn_norm, 1, cfg["rms_eps"],
                                                                     dm.layers[l].wgate, dm.layers[l].wup, y.ptr, F, D),
            lambda l: lib.m40llm_ext_gemv_residual_f32xf16_async(ctx.h, y.ptr, dm.layers[l].wdown, x1.ptr, h.ptr, D, F))
        h.free(); x1.free()
    return out


def measured_traffic(kernel):
    """HBM bytes per launch of the dominant kernel from the committed rocprofv3 --pmc summary (FETCH_SIZE + WRITE_SIZE,
    each scaled by the same counter's reading for a copy of known size); None when no summary covers the kernel."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "decode_b1_tinyllama_traffic.json")
    try:
        with open(path) as f:
            rec = json.load(f)
        return rec.get(kernel, {}).get("hbm_bytes_per_launch")
    except (OSError, ValueError):
        return None


def trace_duration(kernel, key):
    """Average start-to-end duration of a kernel inside the decoded tokens / steps of the committed rocprofv3 kernel
    trace of this same command (profiles/kernel_trace_durations.json), or None."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "kernel_trace_durations.json")
    try:
        with open(path) as f:
            return json.load(f).get(kernel, {}).get(key)
    except (OSError, ValueError):
        return None


def host_cpu():
    """CPU model string and the cores this process may run on."""
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count() or 1
    return model, usable


def cpu_baseline(cfg, W, steps, threads):
    """The CPU oracle (a scalar port of the reference's semantics) timed on this host: `steps` greedy decode
    tokens from an empty KV cache.  At this size a token is bound by the 2.07 GB of weights, not by context."""
    from oracle import pyoracle as orc
    orc.set_threads(threads)
    om = orc.Model(dict(cfg, qkv_bias=bool(cfg.get("qkv_bias"))), W)
    om.alloc_kv(steps + 4, 1)
    t0 = time.perf_counter()
    om.decode_greedy(0, [1], steps)          # 1 prompt token + (steps-1) further forwards + `steps` lm_head passes
    dt = time.perf_counter() - t0
    return dict(value=steps / dt, unit="tok/s", cores=threads, kind="port",
                sample=f"{steps} greedy decode tokens of the same model from an empty KV cache, oracle/oracle.c "
                       f"(gcc -O2{' -fopenmp' if threads > 1 else ''}, {threads} thread{'s' if threads > 1 else ''})")


def cpu_baseline_b8(b8_state, threads, steps=1):
    """The batch-8 half on the CPU: the same Qwen2.5-3B-shaped model, the same eight pre-filled contexts, `steps` greedy
    steps of every sequence with the oracle (sequences one after the other, OpenMP inside each product)."""
    from oracle import pyoracle as orc
    cfg, W, lens, k16, v16, first = b8_state
    orc.set_threads(threads)
    B, L = len(lens), cfg["n_layers"]
    om = orc.Model(dict(cfg, qkv_bias=True), W)
    om.alloc_kv(int(lens.max()) + steps + 2, B)
    Ko, Vo = om.kv_views()
    for s in range(B):
        for l in range(L):
            Ko[s * L + l, :lens[s]] = k16[:lens[s]]; Vo[s * L + l, :lens[s]] = v16[:lens[s]]
    t0 = time.perf_counter()
    for s in range(B):
        om.decode_greedy(s, [int(first[s])], steps, start_pos=int(lens[s]))
    dt = time.perf_counter() - t0
    return dict(value=B * steps / dt, unit="tok/s", cores=threads, kind="port",
                sample=f"{steps} greedy step(s) of the 8 sequences of config.b8 (contexts U[256,4096]), oracle/oracle.c "
                       f"(gcc -O2 -fopenmp, {threads} threads)")


def measure_b8(pkg, syn, ctx, steps=32, warmup=4):
    """The batch-8 half of the metric (BASELINE configs[2]): Qwen2.5-3B-shaped random-init model (36 layers, hidden
    2048, 16 q / 2 kv heads, head_dim 128, FFN 11008, vocab 151936, biases, NeoX RoPE), 8 sequences with contexts
    ~U[256, 4096] pre-filled with N(0,1) K/V, row-batched greedy decode on the fused graph path.  Four distinct random
    layers are repeated over the 36 (each layer has its own device copy, so no layer finds its weights in a cache);
    the embedding table is the lm_head matrix.  Reported beside the batch-1 value, never as it."""
    cfg = dict(syn.QWEN25_3B)
    B = 8
    rng = np.random.default_rng(0)
    lens = rng.integers(256, 4097, size=B).astype(np.uint32)
    W = syn.make_weights(cfg, seed=0, unique_layers=4, tie_embeddings=True)
    dm = syn.DeviceModel(ctx, cfg, W, max_seq_len=4096 + warmup + steps + 8, max_sequences=B)
    dm.set_mode(2)
    f16 = lambda a: np.ascontiguousarray(a.astype(np.float16).view(np.uint16))
    k16h = f16(rng.standard_normal((4096, cfg["kv_heads"], cfg["head_dim"]), dtype=np.float32))
    v16h = f16(rng.standard_normal((4096, cfg["kv_heads"], cfg["head_dim"]), dtype=np.float32))
    dk, dv = ctx.to_device(k16h), ctx.to_device(v16h)
    for s in range(B):
        for l in range(cfg["n_layers"]):
            slot = dm.H.m40host_model_kv_slot(dm.h, s, l)
            pkg.check(ctx.lib.m40llm_ext_kvcache_bulk_fill_f16(ctx.h, dm.kv_handle(), slot, dk.ptr, dv.ptr, int(lens[s])),
                      "m40llm_ext_kvcache_bulk_fill_f16")
    first = rng.integers(0, cfg["vocab"], size=B).astype(np.uint32)
    ids, ms = dm.decode_batch_timed(np.arange(B), lens, first, warmup, steps)
    D, F, V, L = cfg["d_model"], cfg["ffn"], cfg["vocab"], cfg["n_layers"]
    KV = cfg["kv_heads"] * cfg["head_dim"]
    # the dominant kernel of this half: RMSNorm + gate/up + SwiGLU of eight rows in one launch (rows_mfma_kernel<1, 8>),
    # timed inside the chain O projection -> gate/up -> down projection over the layers' own weights
    lib = ctx.lib
    xa = ctx.to_device(np.random.default_rng(2).standard_normal((B, D)).astype(np.float32))
    x1, hid, xo = ctx.alloc(B * D * 4), ctx.alloc(B * F * 4), ctx.alloc(B * D * 4)
    ly = dm.layers
    gate_up_bytes = 2 * F * D * 2 + B * D * 4 + D * 4 + B * F * 4           # two matrices + rows + norm weights in, hidden rows out
    before = lambda l: lib.m40llm_ext_batched_gemm_residual_f32xf16_async(ctx.h, xa.ptr, ly[l].wo, xa.ptr, x1.ptr, B, D, D)
    kernel = lambda l: lib.m40llm_ext_batched_norm_gate_up_swiglu_clear_async(ctx.h, x1.ptr, ly[l].ffn_norm, 1, cfg["rms_eps"],
                                                                             ly[l].wgate, ly[l].wup, hid.ptr, B, F, D, xo.ptr, B * D)
    after = lambda l: lib.m40llm_ext_batched_gemm_residual_onto_zero_f32xf16_async(ctx.h, hid.ptr, ly[l].wdown, x1.ptr, xo.ptr, B, D, F)
    for l in range(L):
        for call, what in ((before, "O projection"), (kernel, "gate/up"), (after, "down projection")):
            pkg.check(call(l), what)
    gate_up_us = chain_cost_us(ctx, L, before, kernel, after)
    e0, e1 = ctx.event(), ctx.event()
    ctx.sync(1); ctx.record(e0, 1)
    for rep in range(3):
        for l in range(L):
            kernel(l)
    ctx.record(e1, 1)
    gate_up_b2b_us = ctx.elapsed_ms(e0, e1) * 1e3 / (3 * L)
    ctx.event_destroy(e0); ctx.event_destroy(e1)
    yard = plain_read_yardstick(pkg, ctx, gate_up_bytes)
    for b in (xa, x1, hid, xo):
        b.free()
    gate_up_traffic = None
    try:
        with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "kernel_counters.json")) as f:
            gate_up_traffic = json.load(f)["decode_b8"]["rows_mfma_kernel<1, 8>@131072"]["hbm_bytes_per_launch"]
    except (OSError, ValueError, KeyError):
        pass
    gate_up_trace_us = trace_duration("rows_mfma_kernel<1, 8>", "in_step_avg_us")
    gate_up_live_us = gate_up_us
    gate_up_us = max(gate_up_live_us, gate_up_trace_us) if gate_up_trace_us else gate_up_live_us
    wbytes = L * 2 * (D * (D + 2 * KV) + D * D + 3 * D * F) + 2 * V * D
    kvbytes = int(lens.sum() + B * (warmup + steps / 2)) * L * KV * 2 * 2
    fallback = dm.last_timed_host_fallback()
    dm.close()
    dk.free(); dv.free()
    ms_step = ms / steps
    rec = {"workload": "Qwen2.5-3B-shaped random-init decode (BASELINE configs[2]), batch 8, contexts U[256,4096], "
                       "row-batched greedy, fused + graph", "tok_s": B * steps / (ms / 1e3), "ms_per_step": ms_step,
           "steps": steps, "warmup": warmup, "algorithmic_bytes_per_step": int(wbytes + kvbytes),
           "whole_step_hbm_frac": (wbytes + kvbytes) / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
           "host_sampler_fallback": fallback,
           "roofline": {"bound": "hbm", "kernel": "rows_mfma_kernel<1, 8>", "shape": f"M={B} N=2x{F} K={D}",
                        "algorithmic_bytes_per_launch": gate_up_bytes,
                        "achieved": gate_up_bytes / (gate_up_us * 1e-6) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": gate_up_bytes / (gate_up_us * 1e-6) / 1e9 / HBM_PEAK_GBS,
                        # avg_launch_us (what achieved and frac follow from): the larger of in_chain_us -- live: the chain O
                        # projection -> gate/up -> down projection over the layers, with minus without the kernel, per layer -- and
                        # trace_in_step_us, the kernel's start-to-end time inside the steps of the committed rocprofv3 trace;
                        # back_to_back_us: launches of this kernel alone, one after the other
                        "avg_launch_us": gate_up_us, "in_chain_us": gate_up_live_us, "trace_in_step_us": gate_up_trace_us,
                        "trace_source": "profiles/kernel_trace_durations.json", "back_to_back_us": gate_up_b2b_us,
                        "plain_read_us": yard["us"], "plain_read_workgroups": yard["workgroups"],
                        "frac_of_plain_read": yard["us"] / gate_up_us,
                        # HBM bytes per launch from the committed rocprofv3 --pmc summary (FETCH_SIZE + WRITE_SIZE, scaled by a copy
                        # of known size): not a quantity of this run
                        "traffic": gate_up_traffic, "traffic_source": "profiles/kernel_counters.json (decode_b8)"}}
    return rec, (cfg, W, lens, k16h, v16h, first)


def measure_prefill(syn, ctx, cfg, W, tokens=4096, reps=3):
    """The step before decode, reported beside the metric (never folded into value): one prompt of `tokens` ids through
    the packed prefill forward of the same model (all layers, last-token logits), host clock around the blocking call."""
    dm = syn.DeviceModel(ctx, cfg, W, max_seq_len=tokens + 8, max_sequences=1)
    dm.set_mode(2)
    prompt = np.random.default_rng(1).integers(0, cfg["vocab"], size=tokens).tolist()
    dm.forward_prefill([0], [prompt])
    t0 = time.perf_counter()
    for _ in range(reps):
        dm.forward_prefill([0], [prompt])
    ms = (time.perf_counter() - t0) * 1e3 / reps
    dm.close()
    return {"workload": f"one prompt of {tokens} tokens, packed prefill forward of the same {cfg['n_layers']}-layer model, "
                        "last-token logits included", "prompt_tokens": tokens, "ms": ms, "tok_s": tokens / (ms * 1e-3), "runs_timed": reps}


def plain_read_yardstick(pkg, ctx, nbytes):
    """Fastest of a few workgroup counts for a plain one-launch read of nbytes (rotating over cold buffers): what a
    bandwidth-bound kernel of this size can reach on this box, launch ramp and tail included."""
    nbuf = int(max(2, min(24, (1 << 30) // nbytes)))
    bufs = [ctx.alloc(nbytes) for _ in range(nbuf)]
    out = ctx.alloc(2048 * 4)
    e0, e1 = ctx.event(), ctx.event()
    best = None
    for wgs in (256, 512, 1024, 2048, 4096):
        reps = 3 * nbuf
        for i in range(nbuf + reps):
            if i == nbuf:
                ctx.sync(1)
                ctx.record(e0, 1)
            pkg.check(ctx.lib.m40llm_ext_read_probe_async(ctx.h, bufs[i % nbuf].ptr, nbytes, wgs, out.ptr),
                      "m40llm_ext_read_probe_async")
        ctx.record(e1, 1)
        us = ctx.elapsed_ms(e0, e1) * 1e3 / reps
        if best is None or us < best["us"]:
            best = {"us": us, "workgroups": wgs}
    for b in bufs:
        b.free()
    out.free()
    return best


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--mode", type=int, default=int(os.environ.get("M40_BENCH_MODE", "-1")),
                    help="-1 best available, 0 reference call sequence, 1 fused, 2 fused + graph")
    ap.add_argument("--layers", type=int, default=0, help="override the layer count (debug only; invalidates the metric)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-steps", type=int, default=48)
    ap.add_argument("--kernel-reps", type=int, default=10)
    ap.add_argument("--no-b8", action="store_true", help="skip the batch-8 measurement reported in config.b8")
    ap.add_argument("--no-prefill", action="store_true", help="skip the packed-prefill measurement reported in config.prefill")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also run one 256 MiB device-to-device copy through the library (calibrates rocprofv3 --pmc "
                         "FETCH_SIZE / WRITE_SIZE readings against a transfer of known size)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU form (each box has one MI355X); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import torch
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    pkg = importlib.import_module("m40-llm_amd")
    if not (os.path.exists(pkg.NATIVE_LIB) and os.path.exists(pkg.HOST_LIB)):
        pkg.build()                      # nothing built in this tree: build once; otherwise load what is there
    syn = importlib.import_module("m40-llm_amd.synthetic")

    cfg = dict(syn.TINYLLAMA_1B)
    if args.layers:
        cfg["n_layers"] = args.layers
    n_prompt = 32
    max_seq = n_prompt + args.warmup + args.steps + 8
    t_setup = time.perf_counter()
    W = syn.make_weights(cfg, seed=0)
    ctx = pkg.Context(0)
    dm = syn.DeviceModel(ctx, cfg, W, max_seq_len=max_seq, max_sequences=1)
    mode = args.mode
    if mode < 0:
        mode = 2
    dm.set_mode(mode)
    prompt = np.random.default_rng(0).integers(0, cfg["vocab"], size=n_prompt).astype(np.uint32)
    setup_s = time.perf_counter() - t_setup

    torch.cuda.synchronize()
    ids, elapsed_ms = dm.decode_timed(0, prompt, args.warmup, args.steps)     # timed region brackets itself with full syncs
    torch.cuda.synchronize()
    tok_s = args.steps / (elapsed_ms / 1e3)
    ms_per_step = elapsed_ms / args.steps

    if args.traffic_probe:
        n = 256 << 20
        src, dst = ctx.alloc(n), ctx.alloc(n)
        for _ in range(3):
            pkg.check(ctx.lib.m40llm_memcpy_d2d_async(ctx.h, dst.ptr, src.ptr, n, 1), "m40llm_memcpy_d2d_async")
        ctx.sync(1)
        src.free(); dst.free()
    dom = measure_dominant_kernel(pkg, ctx, dm, cfg, args.kernel_reps, mode)
    # The kernel's duration inside a token: live, from the chain of launches it depends on (chain with minus chain
    # without); launches of the kernel alone, back to back, overlap their ramps and read faster (kept as back_to_back_*).
    # The committed kernel trace of this command gives the kernel's own start-to-end time inside graph-replayed tokens;
    # the chain difference can hide part of the kernel behind its neighbours, so the larger of the two is what achieved
    # and frac are computed from.
    trace_us = trace_duration(dom["kernel"], "in_token_avg_us")
    live_us = dom["in_chain_us"] or dom["avg_us"]
    dom_us = max(live_us, trace_us) if trace_us else live_us
    achieved = dom["bytes"] / (dom_us * 1e-6) / 1e9
    yard = plain_read_yardstick(pkg, ctx, dom["bytes"])
    token_bytes = algorithmic_bytes_per_token(cfg)
    out = {
        "metric": "decode tok/s at B=1 and B=8; attn+GEMV HBM GB/s as % of MI355X peak",
        "value": tok_s, "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "TinyLlama-1.1B-shaped random-init dense decode (BASELINE configs[1]): 22 layers, hidden 2048, "
                               "32 q / 4 kv heads, head_dim 64, FFN 5632, vocab 32000, f16 weights N(0,0.02), 32 random prompt "
                               "ids, greedy decode, batch 1",
                   "batch": 1, "prompt_tokens": n_prompt, "layers": cfg["n_layers"],
                   "host_path": ["reference call sequence", "fused", "fused + graph"][mode],
                   "whole_step_hbm_gbs": token_bytes / (ms_per_step * 1e-3) / 1e9,
                   "whole_step_hbm_frac": token_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
                   "algorithmic_bytes_per_token": token_bytes, "setup_s": round(setup_s, 1),
                   "first_generated_ids": [int(i) for i in ids[n_prompt:n_prompt + 8]]},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": measured_traffic(dom["kernel"]),
                     # not a quantity of this run: read from the committed counter summary of an earlier profiled run
                     "traffic_source": "profiles/decode_b1_tinyllama_traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, "
                                       "collected beforehand with the same command under the profiler)",
                     "kernel": dom["kernel"], "shape": dom["shape"],
                     # avg_launch_us: what achieved / frac are computed from: the larger of in_chain_us (live: the chain O
                     # projection -> this kernel -> down projection over all layers between one pair of events, minus the same
                     # chain without it, per layer) and trace_in_token_us (the kernel's start-to-end time inside the decoded
                     # tokens of the committed rocprofv3 trace of this command).  back_to_back_us: launches of this kernel alone,
                     # one after the other (their ramps overlap).  event_pair_us: one event pair around every launch inside
                     # that chain (includes the wait for the launch before)
                     "avg_launch_us": dom_us, "launches_timed": dom["launches"],
                     "in_chain_us": live_us, "trace_in_token_us": trace_us,
                     "trace_source": "profiles/kernel_trace_durations.json (rocprofv3 --kernel-trace of this command, collected beforehand)",
                     "back_to_back_us": dom["avg_us"],
                     "back_to_back_frac": dom["bytes"] / (dom["avg_us"] * 1e-6) / 1e9 / HBM_PEAK_GBS,
                     "event_pair_us": dom["in_token_us"],
                     "algorithmic_bytes_per_launch": dom["bytes"],
                     # a kernel that only reads the same number of bytes, one launch, fastest of five grid sizes
                     "plain_read_us": yard["us"], "plain_read_workgroups": yard["workgroups"],
                     "frac_of_plain_read": yard["us"] / dom_us},
    }
    out["config"]["host_sampler_fallback"] = dm.last_timed_host_fallback()
    dm.close()
    if not args.no_prefill and not args.layers:
        try:
            out["config"]["prefill"] = measure_prefill(syn, ctx, cfg, W)
        except Exception as e:
            out["config"]["prefill"] = {"error": repr(e)}
    b8_state = None
    if not args.no_b8 and not args.layers:
        try:
            out["config"]["b8"], b8_state = measure_b8(pkg, syn, ctx)
        except Exception as e:     # the batch-1 line must still be printed
            out["config"]["b8"] = {"error": repr(e)}
    if not args.no_cpu_baseline:
        model, usable = host_cpu()
        threads = max(1, min(usable, 16))       # the GPU box gives one GPU's share of its cores: 16
        base = cpu_baseline(cfg, W, args.cpu_steps, 1)
        base["cpu_model"] = model
        base["usable_cores"] = usable
        variants = []
        try:
            variants.append(dict(cpu_baseline(cfg, W, 2 * args.cpu_steps, threads), workload="batch 1 (the headline workload), OpenMP"))
            if b8_state is not None:
                variants.append(dict(cpu_baseline_b8(b8_state, threads), workload="batch 8 (config.b8), OpenMP"))
        except Exception as e:
            variants.append({"error": repr(e)})
        base["variants"] = variants
        out["cpu_baseline"] = base
    print(json.dumps(out))


if __name__ == "__main__":
    main()
