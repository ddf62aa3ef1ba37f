"""Per-kernel throughput of the decode hot path on one MI355X, against the HBM roofline.

    python m40-llm_amd/kernel_bench.py [--only read,attn,gemv,gemm8,q80,bsel,decode8,prefill,gguf,pfwd,gemmN,sched] [--json out.jsonl]

Every case launches through the C-ABI library on its decode (or prefill) stream and is timed with
events recorded on that same stream: `reps` launches between two events, inputs rotated over enough
distinct buffers that no launch finds its operands in a cache left warm by the previous one (a decode
step never re-reads a weight or a KV row within a token).  "GB/s" is algorithmic bytes (the minimum
traffic of the operation) divided by the average launch time; "frac" is that over 8 TB/s.
"""
from __future__ import annotations

import argparse
import importlib
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
m40 = importlib.import_module("m40-llm_amd")

PEAK_GBS = 8000.0


class Bench:
    def __init__(self):
        self.ctx = m40.Context(0)
        self.lib = self.ctx.lib
        self.h = self.ctx.h
        self.rows = []
        self.e0, self.e1 = self.ctx.event(), self.ctx.event()

    def call(self, name, *args):
        rc = getattr(self.lib, name)(self.h, *args)
        if rc != 0:
            raise m40.M40Error(name, rc)

    def time(self, name, shape, algo_bytes, launch, n_variants, stream=1, reps=None, warm=None, quiet=False):
        """launch(i) enqueues one launch on variant i; returns microseconds per launch."""
        reps = reps or max(2 * n_variants, 64)
        warm = warm or max(n_variants, 8)
        for i in range(warm):
            launch(i % n_variants)
        self.ctx.sync(0); self.ctx.sync(1)
        self.ctx.record(self.e0, stream)
        for i in range(reps):
            launch(i % n_variants)
        self.ctx.record(self.e1, stream)
        ms = self.ctx.elapsed_ms(self.e0, self.e1)
        us = ms * 1e3 / reps
        gbs = algo_bytes / us / 1e3
        row = dict(kernel=name, shape=shape, us_per_launch=round(us, 3), algorithmic_bytes=int(algo_bytes),
                   gbs=round(gbs, 1), frac=round(gbs / PEAK_GBS, 4), launches=reps, buffers=n_variants)
        self.rows.append(row)
        if not quiet:
            print(f"{name:34s} {shape:44s} {us:9.2f} us {gbs:8.1f} GB/s  frac {gbs / PEAK_GBS:6.3f}", flush=True)
        return us


def f16(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32).astype(np.float16).view(np.uint16))


def n_rot(nbytes, budget=3 << 30, cap=64):
    return int(max(2, min(cap, budget // max(nbytes, 1))))


def bench_attention(b: Bench):
    rng = np.random.default_rng(0)
    # dense last-token GQA attention: config 1 shape, and the same heads at longer contexts
    for qh, kvh, hd, L in ((32, 4, 64, 128), (32, 4, 64, 512), (32, 4, 64, 4096), (16, 2, 128, 4096), (32, 8, 128, 32768)):
        kv_bytes = L * kvh * hd * 2 * 2
        nseq = n_rot(kv_bytes, budget=2 << 30, cap=32)
        kv = m40.KVCache(b.ctx, L, nseq, kvh, hd)
        k = f16(rng.standard_normal((L, kvh, hd))); v = f16(rng.standard_normal((L, kvh, hd)))
        dk, dv = b.ctx.to_device(k), b.ctx.to_device(v)
        for s in range(nseq):
            b.call("m40llm_ext_kvcache_bulk_fill_f16", kv.h, s, dk.ptr, dv.ptr, L)
        q = b.ctx.to_device(rng.standard_normal(qh * hd).astype(np.float32))
        out = b.ctx.alloc(qh * hd * 4)
        algo = kv_bytes + 2 * qh * hd * 4
        b.time("attention_last_token_gqa", f"qh{qh} kvh{kvh} hd{hd} L{L}", algo,
               lambda i: b.call("m40llm_attention_last_token_f32_gqa_async", kv.h, i, q.ptr, qh, L, out.ptr), nseq)
        kv.destroy()
    # row-batched variable-length attention: config 3 shape
    qh, kvh, hd, B, maxL = 16, 2, 128, 8, 4160
    lens = rng.integers(256, 4097, size=B).astype(np.uint32)
    nset = 4
    kv = m40.KVCache(b.ctx, maxL, B * nset, kvh, hd)
    k = f16(rng.standard_normal((maxL, kvh, hd))); dk = b.ctx.to_device(k)
    for s in range(B * nset):
        b.call("m40llm_ext_kvcache_bulk_fill_f16", kv.h, s, dk.ptr, dk.ptr, int(lens[s % B]))
    q = b.ctx.to_device(rng.standard_normal((B, qh * hd)).astype(np.float32))
    out = b.ctx.alloc(B * qh * hd * 4)
    dl = b.ctx.to_device(lens)
    ids = [b.ctx.to_device((np.arange(B) + B * i).astype(np.uint32)) for i in range(nset)]
    algo = int(lens.sum()) * kvh * hd * 2 * 2 + 2 * B * qh * hd * 4
    b.time("attention_gqa_batched", f"B8 qh16 kvh2 hd128 lens U[256,4096] sum {int(lens.sum())}", algo,
           lambda i: b.call("m40llm_attention_last_token_f32_gqa_batched_async", kv.h, ids[i].ptr, dl.ptr, B, q.ptr, qh,
                            out.ptr), nset)
    lens_m1 = b.ctx.to_device((lens - 1).astype(np.uint32))
    b.time("attention_gqa_batched (lens on device)", f"B8 qh16 kvh2 hd128 lens U[256,4096] sum {int(lens.sum())}", algo,
           lambda i: b.call("m40llm_ext_attention_last_token_f32_gqa_batched_lens_dev_async", kv.h, ids[i].ptr, lens_m1.ptr, 1, B,
                            4096, q.ptr, qh, out.ptr), nset)
    kv.destroy()


def bench_read_probe(b: Bench):
    """Plain read of N bytes in one launch: what a bandwidth-bound kernel of that size can at best reach on this box."""
    out = b.ctx.alloc(2048 * 4)
    for label, nbytes in (("O projection weights (TinyLlama)", 2048 * 2048 * 2), ("down weights (TinyLlama)", 2048 * 5632 * 2),
                          ("gate + up weights (TinyLlama)", 2 * 2048 * 5632 * 2), ("gate + up weights (Qwen2.5-3B)", 2 * 2048 * 11008 * 2),
                          ("lm_head weights (TinyLlama)", 32000 * 2048 * 2), ("K + V, 32768 tokens x 8 heads x 128", 32768 * 8 * 128 * 2 * 2)):
        nbuf = n_rot(nbytes, budget=2 << 30, cap=48)
        bufs = [b.ctx.alloc(nbytes) for _ in range(nbuf)]
        best = None
        for wgs in (256, 512, 1024, 2048, 4096, 8192):          # the fastest split is the yardstick
            rows_before = len(b.rows)
            us = b.time("plain read, one launch", f"{label}: {nbytes / 1e6:.1f} MB, {wgs} workgroups", nbytes,
                        lambda i: b.call("m40llm_ext_read_probe_async", bufs[i].ptr, nbytes, wgs, out.ptr), nbuf, quiet=True)
            row = b.rows.pop(rows_before)
            if best is None or us < best["us_per_launch"]:
                best = row
        b.rows.append(best)
        print(f"{best['kernel']:34s} {best['shape']:44s} {best['us_per_launch']:9.2f} us {best['gbs']:8.1f} GB/s  frac {best['frac']:6.3f}",
              flush=True)
        for x in bufs:
            x.free()


PEAK_F16_MATRIX_TFLOPS = 2500.0


def bench_prefill(b: Bench):
    """Packed variable-length causal prefill attention (f32 in and out): arithmetic-bound.  Useful flops = 4 * head_dim
    per visible (query, key) pair and q head; every product is three f16 matrix instructions on exact two-part splits
    of its f32 operands, so the issued rate is three times the useful one and is what the 2.5 PFLOP/s f16 peak bounds."""
    rng = np.random.default_rng(0)
    cases = [("qh32 kvh4 hd64, one sequence of 512", 32, 4, 64, [512]), ("qh32 kvh4 hd64, one sequence of 4096", 32, 4, 64, [4096]),
             ("qh16 kvh2 hd128, one sequence of 4096", 16, 2, 128, [4096]),
             ("qh16 kvh2 hd128, 8 sequences U[256,4096]", 16, 2, 128, [int(x) for x in rng.integers(256, 4097, size=8)])]
    for label, qh, kvh, hd, lens in cases:
        n = sum(lens)
        q = b.ctx.to_device(rng.standard_normal((n, qh, hd), dtype=np.float32))
        k = b.ctx.to_device(rng.standard_normal((n, kvh, hd), dtype=np.float32))
        v = b.ctx.to_device(rng.standard_normal((n, kvh, hd), dtype=np.float32))
        out = b.ctx.alloc(n * qh * hd * 4)
        lens_np = np.asarray(lens, dtype=np.uint32)
        offs = np.concatenate([[0], np.cumsum(lens_np)[:-1]]).astype(np.uint32)
        dl, do = b.ctx.to_device(lens_np), b.ctx.to_device(offs)
        pairs = sum(L * (L + 1) // 2 for L in lens)
        flops = 4.0 * hd * pairs * qh
        reps, warm = 6, 2
        for i in range(warm + reps):
            if i == warm:
                b.ctx.sync(0)
                b.ctx.record(b.e0, 0)
            b.call("m40llm_attention_prefill_f32_gqa_varlen_async", q.ptr, k.ptr, v.ptr, do.ptr, do.ptr, dl.ptr, dl.ptr, len(lens), qh, kvh,
                   hd, out.ptr)
        b.ctx.record(b.e1, 0)
        us = b.ctx.elapsed_ms(b.e0, b.e1) * 1e3 / reps
        tf = flops / us / 1e6
        b.rows.append(dict(kernel="attention_prefill_gqa_varlen", shape=label, us_per_launch=round(us, 2), flops=flops,
                           useful_tflops=round(tf, 2), issued_tflops=round(3 * tf, 2),
                           frac_f16_matrix_peak=round(3 * tf / PEAK_F16_MATRIX_TFLOPS, 4), launches=reps))
        print(f"{'attention_prefill_gqa_varlen':34s} {label:44s} {us:9.1f} us {tf:8.1f} TFLOP/s useful, {3 * tf:7.1f} issued  "
              f"frac {3 * tf / PEAK_F16_MATRIX_TFLOPS:6.3f} of the f16 matrix peak", flush=True)
        for x in (q, k, v, out, dl, do):
            x.free()


def bench_gguf_load(b: Bench):
    """Weight-file ingestion: a TinyLlama-1.1B-shaped f16 GGUF file (synthetic weights, ~2.2 GB) from the page cache
    into HBM through m40host_gguf_load (parse + validate + streamed upload), beside the reference's sequence on the
    same file (read the whole file into host memory, then m40llm_upload_weights; src/infer/load.rs:11-40), and the
    decode rate of a model assembled from the loaded file.  Bound: the host-to-device link, not HBM."""
    import ctypes as C
    import tempfile
    import time
    gg = importlib.import_module("m40-llm_amd.gguf")
    syn = importlib.import_module("m40-llm_amd.synthetic")
    cfg = dict(syn.TINYLLAMA_1B, context_length=2048)
    W = syn.make_weights(cfg, seed=0, unique_layers=2)
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "tinyllama_shape_f16.gguf")
        size = gg.write_model_file(path, cfg, W)
        del W
        times = []
        for _ in range(3):
            t0 = time.perf_counter()
            gw = gg.GgufWeights(b.ctx, path)
            times.append(time.perf_counter() - t0)
            if len(times) < 3:
                gw.close()
        best = min(times)
        t0 = time.perf_counter()
        blob = np.fromfile(path, dtype=np.uint8)
        p = C.c_void_p()
        m40.check(b.lib.m40llm_upload_weights(b.ctx.h, blob.ctypes.data_as(C.c_void_p), blob.nbytes, C.byref(p)), "m40llm_upload_weights")
        t_ref = time.perf_counter() - t0
        b.lib.m40llm_device_free(b.ctx.h, p)
        del blob
        gm = gw.model(max_seq_len=256, max_sequences=1)
        gm.set_mode(2)
        ids, ms = gm.decode_timed(0, [1, 2, 3, 4], 8, 64)
        gm.close()
        gw.close()
    row = dict(kernel="gguf load (parse, validate, streamed upload)", shape=f"TinyLlama-1.1B shape, f16, {size / 1e9:.2f} GB file",
               seconds=round(best, 4), gb_per_s=round(size / best / 1e9, 2), read_then_upload_seconds=round(t_ref, 4),
               read_then_upload_gb_per_s=round(size / t_ref / 1e9, 2), decode_tok_s_from_file=round(64e3 / ms, 1))
    b.rows.append(row)
    print(f"{'gguf load':34s} {row['shape']:44s} {best * 1e3:9.1f} ms {row['gb_per_s']:8.2f} GB/s file->HBM   "
          f"(read whole file + upload_weights: {t_ref * 1e3:.1f} ms, {row['read_then_upload_gb_per_s']:.2f} GB/s); "
          f"decode from the loaded file {row['decode_tok_s_from_file']:.1f} tok/s", flush=True)


def bench_gemm_many_rows(b: Bench):
    """The many-row GEMM of the prefill path (f32 activations split into two f16 parts: two matrix instructions per
    product tile).  Useful rate = 2 M N K / time; the instruction rate is twice that and is what the 2.5 PFLOP/s f16
    peak bounds."""
    rng = np.random.default_rng(3)
    for M, N, K in ((4096, 2048, 2048), (4096, 256, 2048), (4096, 5632, 2048), (4096, 2048, 5632), (512, 5632, 2048), (16384, 11008, 2048)):
        A = b.ctx.to_device(rng.standard_normal((M, K), dtype=np.float32))
        W = b.ctx.to_device(f16(rng.standard_normal((N, K), dtype=np.float32) * 0.02))
        Cb = b.ctx.alloc(M * N * 4)
        reps, warm = 10, 2
        for i in range(warm + reps):
            if i == warm:
                b.ctx.sync(1)
                b.ctx.record(b.e0, 1)
            b.call("m40llm_ext_gemm_f32xf16_gguf_f32_async", A.ptr, W.ptr, Cb.ptr, M, N, K, 1)
        b.ctx.record(b.e1, 1)
        us = b.ctx.elapsed_ms(b.e0, b.e1) * 1e3 / reps
        tf = 2.0 * M * N * K / us / 1e6
        b.rows.append(dict(kernel="gemm_f32xf16_gguf many rows", shape=f"M={M} N={N} K={K}", us_per_launch=round(us, 2),
                           useful_tflops=round(tf, 1), instruction_tflops=round(2 * tf, 1),
                           frac_f16_matrix_peak=round(2 * tf / PEAK_F16_MATRIX_TFLOPS, 4)))
        print(f"{'gemm_f32xf16_gguf many rows':34s} {f'M={M} N={N} K={K}':44s} {us:9.1f} us {tf:8.1f} TFLOP/s useful, {2 * tf:7.1f} issued  "
              f"frac {2 * tf / PEAK_F16_MATRIX_TFLOPS:6.3f} of the f16 matrix peak", flush=True)
        for x in (A, W, Cb):
            x.free()


def bench_prefill_forward(b: Bench):
    """Whole prefill forward (every layer, packed prompts) of the TinyLlama-1.1B shape through the host layer:
    tokens per second and the matrix-instruction rate of the projections (2 * rows * weight elements per layer;
    f16 instructions on hi/lo-split f32 activations, so the bound is half the 2.5 PFLOP/s f16 peak)."""
    import time
    syn = importlib.import_module("m40-llm_amd.synthetic")
    cfg = dict(syn.TINYLLAMA_1B)
    W = syn.make_weights(cfg, seed=0, unique_layers=2)
    dm = syn.DeviceModel(b.ctx, cfg, W, max_seq_len=4096, max_sequences=8)
    del W
    rng = np.random.default_rng(0)
    per_layer = cfg["d_model"] * (2 * cfg["d_model"] + 2 * cfg["kv_heads"] * cfg["head_dim"] + 3 * cfg["ffn"])
    for label, lens in (("one prompt of 512", [512]), ("one prompt of 4096", [4096]), ("8 prompts U[256,4096]", [int(x) for x in rng.integers(256, 4097, size=8)])):
        prompts = [rng.integers(0, cfg["vocab"], size=n).tolist() for n in lens]
        seqs = list(range(len(lens)))
        dm.forward_prefill(seqs, prompts, want_logits=False)          # warm (workspace, tables)
        t0 = time.perf_counter()
        dm.forward_prefill(seqs, prompts, want_logits=False)
        dt = time.perf_counter() - t0
        rows = sum(lens)
        tf = 2.0 * rows * per_layer * cfg["n_layers"] / dt / 1e12
        b.rows.append(dict(kernel="prefill forward, TinyLlama-1.1B shape", shape=label, rows=rows, ms=round(dt * 1e3, 2),
                           tok_s=round(rows / dt, 1), projection_tflops=round(tf, 1)))
        print(f"{'prefill forward (22 layers)':34s} {label:44s} {dt * 1e3:9.1f} ms {rows / dt:10.0f} tok/s   projections {tf:6.1f} TFLOP/s", flush=True)
    dm.close()


def bench_scheduler(b: Bench):
    """Continuous batching end to end (TinyLlama-1.1B shape, synthetic weights): 32 requests with prompts of 64-512
    tokens and 64 new tokens each through 8 sequence slots, host-sampled greedy; beside the same requests served one
    after the other on one slot."""
    import time
    syn = importlib.import_module("m40-llm_amd.synthetic")
    sch = importlib.import_module("m40-llm_amd.scheduler")
    cfg = dict(syn.TINYLLAMA_1B)
    W = syn.make_weights(cfg, seed=0, unique_layers=2, std=0.02, emb_std=1.0)
    dm = syn.DeviceModel(b.ctx, cfg, W, max_seq_len=1024, max_sequences=8)
    del W
    dm.set_mode(2)
    rng = np.random.default_rng(1)
    reqs = [rng.integers(0, cfg["vocab"], size=int(n)).tolist() for n in rng.integers(64, 513, size=32)]
    new_tokens = 64
    for label, slots in (("8 slots, continuous batching", 8), ("1 slot, one request at a time", 1)):
        s = sch.Scheduler.for_model(dm, slots)
        pending = list(reqs)
        warm = s.submit(reqs[0][:16], max_tokens=4)          # graph capture, workspaces
        s.run_until_idle()
        assert s.state(warm) == "complete"
        t0 = time.perf_counter()
        ticks = 0
        while pending or s.active():
            while pending and s.available_slots():
                s.submit(pending.pop(0), max_tokens=new_tokens)
            s.tick()
            ticks += 1
        dt = time.perf_counter() - t0
        gen = len(reqs) * new_tokens
        prompt_tokens = sum(len(r) for r in reqs)
        b.rows.append(dict(kernel="decode scheduler, TinyLlama-1.1B shape", shape=label, requests=len(reqs), prompt_tokens=prompt_tokens,
                           generated=gen, seconds=round(dt, 3), generated_tok_s=round(gen / dt, 1), ticks=ticks))
        print(f"{'decode scheduler':34s} {label:44s} {dt * 1e3:9.1f} ms {gen / dt:10.1f} generated tok/s   ({len(reqs)} requests, "
              f"{prompt_tokens} prompt tokens, {ticks} ticks)", flush=True)
        s.close()
    dm.close()


def bench_gemv(b: Bench, M: int):
    rng = np.random.default_rng(1)
    shapes = [(2048, 2048), (256, 2048), (5632, 2048), (2048, 5632), (32000, 2048)] if M == 1 else \
             [(2048, 2048), (256, 2048), (11008, 2048), (2048, 11008), (151936, 2048)]
    for N, K in shapes:
        wbytes = N * K * 2
        nb = n_rot(wbytes, budget=3 << 30, cap=48)
        w = f16(rng.standard_normal((N, K)) * 0.02)
        bufs = [b.ctx.to_device(w) for _ in range(nb)]
        a = b.ctx.to_device(rng.standard_normal((M, K)).astype(np.float32))
        c = b.ctx.alloc(M * N * 4)
        algo = wbytes + M * K * 4 + M * N * 4
        b.time(f"gemm_f32xf16_gguf M={M}", f"N={N} K={K}", algo,
               lambda i: b.call("m40llm_ext_gemm_f32xf16_gguf_f32_async", a.ptr, bufs[i].ptr, c.ptr, M, N, K, 1), nb)
        for x in bufs:
            x.free()


def bench_q80(b: Bench):
    rng = np.random.default_rng(2)
    d_model, ffn = 4096, 14336

    def q80(n, k):
        blocks = n * k // 32
        raw = np.zeros((blocks, 34), dtype=np.uint8)
        raw[:, :2] = rng.uniform(0.001, 0.01, blocks).astype(np.float16).view(np.uint8).reshape(blocks, 2)
        raw[:, 2:] = rng.integers(-127, 128, size=(blocks, 32)).astype(np.int8).view(np.uint8)
        return raw
    gate, up, down = q80(ffn, d_model), q80(ffn, d_model), q80(d_model, ffn)
    nset = 6
    sets = [(b.ctx.to_device(gate), b.ctx.to_device(up), b.ctx.to_device(down)) for _ in range(nset)]
    wbytes = gate.nbytes + up.nbytes + down.nbytes
    for M in (1, 2, 4, 8, 16):
        x = b.ctx.to_device(rng.standard_normal((M, d_model)).astype(np.float32))
        scratch = b.ctx.alloc(2 * M * ffn * 4)
        out = b.ctx.alloc(M * d_model * 4)
        algo = wbytes + M * (d_model * 4 * 2)
        b.time("ffn_swiglu_q80", f"M={M} d_model 4096 ffn 14336", algo,
               lambda i: b.call("m40llm_ext_ffn_swiglu_q80_f32_async", x.ptr, sets[i][0].ptr, sets[i][1].ptr, sets[i][2].ptr,
                                scratch.ptr, out.ptr, M, d_model, ffn), nset)
    for M in (1, 2, 4, 8, 16):
        a = b.ctx.to_device(rng.standard_normal((M, d_model)).astype(np.float32))
        c = b.ctx.alloc(M * ffn * 4)
        b.time(f"gemm_f32xq80_gguf M={M}", "N=14336 K=4096", gate.nbytes,
               lambda i: b.call("m40llm_ext_gemm_f32xq80_gguf_f32_async", a.ptr, sets[i][0].ptr, c.ptr, M, ffn, d_model, 1), nset)
        a2 = b.ctx.to_device(rng.standard_normal((M, ffn)).astype(np.float32))
        b.time(f"gemm_f32xq80_gguf M={M}", "N=4096 K=14336", down.nbytes,
               lambda i: b.call("m40llm_ext_gemm_f32xq80_gguf_f32_async", a2.ptr, sets[i][2].ptr, c.ptr, M, d_model, ffn, 1), nset)


def bench_block_select(b: Bench):
    import ctypes as C
    qh, kvh, hd, L, bs, top, W = 32, 8, 128, 32768, 64, 64, 512
    nseq = 4
    old = L - W
    # old V: the reference's q4 (one f32 scale per token and head) and the groups-of-32 scale + min format (backing 3)
    for backing, label, vbytes in ((2, "fp16-K/q4-V", hd // 2 + 4), (3, "fp16-K/q4-V groups of 32", hd // 2 + 4 * (hd // 32))):
        rng = np.random.default_rng(3)
        kv = m40.KVCache(b.ctx, L, nseq, kvh, hd, compressed=dict(recent_window=W, block_size=bs, top_blocks=top,
                                                                  exact_old_backing=backing))
        for s in range(nseq):
            k = f16(rng.standard_normal((L, kvh, hd))); v = f16(rng.standard_normal((L, kvh, hd)))
            dk, dv = b.ctx.to_device(k), b.ctx.to_device(v)
            b.call("m40llm_ext_kvcache_bulk_fill_f16", kv.h, s, dk.ptr, dv.ptr, L)
            dk.free(); dv.free()
        q = b.ctx.to_device(rng.standard_normal(qh * hd).astype(np.float32))
        out = b.ctx.alloc(qh * hd * 4)
        score = old * kvh * hd * 2
        attend = qh * (top * bs * hd * 2 + W * hd * 2 + top * bs * vbytes + W * hd * 2)
        algo = score + attend
        name = "m40llm_attention_last_token_f32_gqa_block_select_exact_fp16_k_q4_v_old_direct_async"
        b.time(f"block_select {label}, B=1", f"qh32 kvh8 hd128 L32768 bs64 top64 W512", algo,
               lambda i: b.call(name, kv.h, i, q.ptr, qh, L, W, bs, top, out.ptr), nseq)

        def four(i):
            for s in range(nseq):
                b.call(name, kv.h, s, q.ptr, qh, L, W, bs, top, out.ptr)
        if backing == 2:
            b.time(f"block_select {label}, B=4", "4 slots per step, one call per slot", 4 * algo, four, 1, reps=16, warm=2)
        q4 = b.ctx.to_device(rng.standard_normal((nseq, qh * hd)).astype(np.float32))
        out4 = b.ctx.alloc(nseq * qh * hd * 4)
        ids_h = np.arange(nseq, dtype=np.uint32); lens_h = np.full(nseq, L, dtype=np.uint32)
        b.time(f"block_select {label}, B=4", "4 slots per step, multi-slot call", 4 * algo,
               lambda i: b.call("m40llm_ext_attention_block_select_fp16_k_q4_v_multi_async", kv.h, nseq,
                                ids_h.ctypes.data_as(C.c_void_p), lens_h.ctypes.data_as(C.c_void_p), q4.ptr, qh, W, bs, top, out4.ptr),
               1, reps=16, warm=2)
        kv.destroy()


def bench_decode_batch(b: Bench, steps=32, warmup=4, mode=2):
    """BASELINE config 3: Qwen2.5-3B-shaped random-init model, 8 sequences with contexts ~U[256, 4096], row-batched
    greedy decode through the host layer.  Four distinct random layers are repeated over the 36 (own device copy
    each); the embedding table is the lm_head matrix."""
    syn = importlib.import_module("m40-llm_amd.synthetic")
    cfg = dict(syn.QWEN25_3B)
    B = 8
    rng = np.random.default_rng(0)
    lens = rng.integers(256, 4097, size=B).astype(np.uint32)
    max_seq = 4096 + warmup + steps + 8
    W = syn.make_weights(cfg, seed=0, unique_layers=4, tie_embeddings=True)
    dm = syn.DeviceModel(b.ctx, cfg, W, max_seq_len=max_seq, max_sequences=B)
    dm.set_mode(mode)
    k16 = f16(rng.standard_normal((4096, cfg["kv_heads"], cfg["head_dim"])))
    v16 = f16(rng.standard_normal((4096, cfg["kv_heads"], cfg["head_dim"])))
    dk, dv = b.ctx.to_device(k16), b.ctx.to_device(v16)
    for s in range(B):
        for l in range(cfg["n_layers"]):
            slot = dm.H.m40host_model_kv_slot(dm.h, s, l)
            b.call("m40llm_ext_kvcache_bulk_fill_f16", dm.kv_handle(), slot, dk.ptr, dv.ptr, int(lens[s]))
    first = rng.integers(0, cfg["vocab"], size=B).astype(np.uint32)
    ids, ms = dm.decode_batch_timed(np.arange(B), lens, first, warmup, steps)
    D, F, V, L = cfg["d_model"], cfg["ffn"], cfg["vocab"], cfg["n_layers"]
    KV = cfg["kv_heads"] * cfg["head_dim"]
    wbytes = L * 2 * (D * (D + 2 * KV) + D * D + 3 * D * F) + 2 * V * D
    kvbytes = int(lens.sum() + B * (warmup + steps / 2)) * L * KV * 2 * 2
    us = ms * 1e3 / steps
    gbs = (wbytes + kvbytes) / us / 1e3
    tok_s = B * steps / (ms / 1e3)
    row = dict(kernel=f"decode step Qwen2.5-3B shape B=8 mode {mode}", shape=f"36 layers, lens sum {int(lens.sum())}", us_per_launch=round(us, 1),
               algorithmic_bytes=int(wbytes + kvbytes), gbs=round(gbs, 1), frac=round(gbs / PEAK_GBS, 4), tok_s=round(tok_s, 1),
               launches=steps, buffers=1)
    b.rows.append(row)
    print(f"{row['kernel']:34s} {row['shape']:44s} {us:9.1f} us {gbs:8.1f} GB/s  frac {gbs / PEAK_GBS:6.3f}  {tok_s:8.1f} tok/s aggregate",
          flush=True)
    dm.close()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--only", default="read,attn,gemv,gemm8,q80,bsel,decode8,prefill,gguf,pfwd,gemmN,sched")
    ap.add_argument("--json", default=None)
    ap.add_argument("--decode-mode", type=int, default=2, help="host path of the decode8 case: 0 reference sequence, 1 fused, 2 fused + graph")
    ap.add_argument("--decode-steps", type=int, default=32, help="timed steps of the decode8 case")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="first copy 256 MiB device-to-device three times through the library: a transfer of known size "
                         "against which rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings of the other kernels are scaled")
    args = ap.parse_args()
    which = set(args.only.split(","))
    b = Bench()
    print(b.lib.m40llm_ext_build_info().decode() if hasattr(b.lib, "m40llm_ext_build_info") else "")
    if args.traffic_probe:
        n = 256 << 20
        src, dst = b.ctx.alloc(n), b.ctx.alloc(n)
        for _ in range(3):
            b.call("m40llm_memcpy_d2d_async", dst.ptr, src.ptr, n, 1)
        b.ctx.sync(1)
        src.free(); dst.free()
    if "read" in which:
        bench_read_probe(b)
    if "attn" in which:
        bench_attention(b)
    if "gemv" in which:
        bench_gemv(b, 1)
    if "gemm8" in which:
        bench_gemv(b, 8)
    if "q80" in which:
        bench_q80(b)
    if "bsel" in which:
        bench_block_select(b)
    if "decode8" in which:
        bench_decode_batch(b, steps=args.decode_steps, mode=args.decode_mode)
    if "prefill" in which:
        bench_prefill(b)
    if "gguf" in which:
        bench_gguf_load(b)
    if "gemmN" in which:
        bench_gemm_many_rows(b)
    if "pfwd" in which:
        bench_prefill_forward(b)
    if "sched" in which:
        bench_scheduler(b)
    if args.json:
        with open(args.json, "w") as f:
            for r in b.rows:
                f.write(json.dumps(r) + "\n")


if __name__ == "__main__":
    main()
