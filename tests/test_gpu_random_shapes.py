"""Seeded sweep over odd shapes: the entry points of the path against the oracle at sizes drawn around the kernels'
tile, chunk and wave boundaries (rows 1-1030, columns 1-5632, K from 8, contexts from 1 token, query blocks of 15-17 and
63-65 and 127-129 queries, cached keys ahead of the queries).  Products are measured in units of the element's own terms
S = sum |a| |w| (2e-6 S: the bound of test_gpu_error_bounds.py with room for the oracle's own rounding), attention
outputs absolutely (|out| <= max |v| ~ 4)."""
import importlib
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(__file__))
from gpu_common import Dev, close, f16bits, m40  # noqa: E402
from test_gpu_block_select import _block_select_case  # noqa: E402
from test_gpu_model import _oracle_greedy_with_logits, _tie_bound  # noqa: E402

syn = importlib.import_module("m40-llm_amd.synthetic")
sch = importlib.import_module("m40-llm_amd.scheduler")

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    return Dev()


def _pick(rng, choices):
    return int(choices[rng.integers(0, len(choices))])


def test_f16_products_at_random_shapes(dev, orc):
    rng = np.random.default_rng(101)
    orc.set_threads(16)
    done = 0
    while done < 60:
        M = _pick(rng, [1, 1, 2, 3, 4, 5, 7, 8, 9, 16, 17, 33, 100, 129, 300, 513, 1030])
        N = _pick(rng, [1, 2, 7, 64, 100, 255, 256, 257, 1000, 2048, 2560, 4097, 5632])
        K = _pick(rng, [8, 16, 24, 32, 64, 72, 256, 1000, 2048, 2056, 4096, 5632])
        if M * N * K > 3e9:
            continue
        A = (rng.standard_normal((M, K)) * (10.0 ** rng.integers(-3, 4))).astype(np.float32)
        B = f16bits(rng.standard_normal((N, K)) * 0.05)
        want = orc.gemm("f32xf16_gguf", A, B, M, N, K)
        got = dev.gemm_gguf(A, B, M, N, K)
        S = np.abs(A).astype(np.float64) @ np.abs(B.view(np.float16).astype(np.float64)).T
        err = float((np.abs(got.astype(np.float64) - want) / (S + 1e-30)).max())
        assert err <= 2e-6, (M, N, K, err)
        done += 1


def test_q80_products_at_random_shapes(dev, orc):
    rng = np.random.default_rng(102)
    orc.set_threads(16)
    done = 0
    while done < 30:
        M = _pick(rng, [1, 2, 3, 4, 5, 8, 9, 16])
        N = _pick(rng, [32, 100, 1000, 4096, 14336])
        K = _pick(rng, [32, 64, 256, 4096, 14336])
        if M * N * K > 1e9:
            continue
        w = np.empty((N, K // 32, 34), dtype=np.uint8)
        w[:, :, :2] = rng.uniform(0.001, 0.01, size=(N, K // 32)).astype(np.float16).view(np.uint8).reshape(N, K // 32, 2)
        w[:, :, 2:] = rng.integers(-127, 128, size=(N, K // 32, 32)).astype(np.int8).view(np.uint8)
        A = rng.standard_normal((M, K)).astype(np.float32)
        want = orc.gemm("f32xq80_gguf", A, w, M, N, K)
        dx, dw, dC = dev.up(A), dev.up(w), dev.zeros(M * N * 4)
        dev.call("m40llm_ext_gemm_f32xq80_gguf_f32", dx.ptr, dw.ptr, dC.ptr, M, N, K)
        got = dC.download(np.float32, (M, N))
        W = (w[:, :, :2].copy().view(np.float16).astype(np.float64) * w[:, :, 2:].view(np.int8).astype(np.float64)).reshape(N, -1)
        S = np.abs(A).astype(np.float64) @ np.abs(W).T
        err = float((np.abs(got.astype(np.float64) - want) / (S + 1e-30)).max())
        assert err <= 2e-6, (M, N, K, err)
        done += 1


def test_dense_attention_at_random_shapes(dev, orc):
    rng = np.random.default_rng(103)
    orc.set_threads(16)
    for _ in range(40):
        hd, kvh, g = _pick(rng, [64, 128]), _pick(rng, [1, 2, 4, 8]), _pick(rng, [1, 2, 4, 8])
        qh = kvh * g
        L = _pick(rng, [1, 2, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 513, 1000, 2049, 4096, 5000])
        K16 = f16bits(rng.standard_normal((L, kvh, hd))).reshape(L, kvh, hd)
        V16 = f16bits(rng.standard_normal((L, kvh, hd))).reshape(L, kvh, hd)
        q = rng.standard_normal(qh * hd).astype(np.float32)
        kv = m40.KVCache(dev.ctx, L, 1, kvh, hd)
        dev.fill_dense(kv, 0, K16, V16)
        got = dev.attention(kv, 0, q, qh, L)
        want = orc.attention(K16[None].copy(), V16[None].copy(), L, kvh, hd, 0, q, qh, L)
        err = float(np.abs(got - want).max())
        assert err <= 2e-5, (qh, kvh, hd, L, err)


def test_packed_prefill_attention_at_random_shapes(dev, orc):
    rng = np.random.default_rng(104)
    orc.set_threads(16)
    done = 0
    while done < 40:
        hd, kvh, g = _pick(rng, [64, 128]), _pick(rng, [1, 2, 4]), _pick(rng, [1, 2, 4, 8])
        qh = kvh * g
        ql = [_pick(rng, [1, 2, 15, 16, 17, 63, 64, 65, 127, 128, 129, 200, 300, 600]) for _ in range(_pick(rng, [1, 2, 3, 5]))]
        kl = [x + _pick(rng, [0, 0, 1, 31, 64, 100]) for x in ql]
        if sum(x * y for x, y in zip(ql, kl)) * qh > 3e7:
            continue
        Q = rng.standard_normal((sum(ql), qh, hd)).astype(np.float32)
        Kf = rng.standard_normal((sum(kl), kvh, hd)).astype(np.float32)
        Vf = rng.standard_normal((sum(kl), kvh, hd)).astype(np.float32)
        rc, want = orc.attention_prefill(Q, Kf, Vf, ql, kl, qh, kvh, hd)
        assert rc == 0
        dq, dk, dv = dev.up(Q), dev.up(Kf), dev.up(Vf)
        dqo, dko = dev.up(orc.prefill_offsets(ql)), dev.up(orc.prefill_offsets(kl))
        dql, dkl = dev.up(np.asarray(ql, dtype=np.uint32)), dev.up(np.asarray(kl, dtype=np.uint32))
        out = dev.zeros(Q.nbytes)
        dev.call("m40llm_attention_prefill_f32_gqa_varlen", dq.ptr, dk.ptr, dv.ptr, dqo.ptr, dko.ptr, dql.ptr, dkl.ptr, len(ql), qh, kvh,
                 hd, out.ptr)
        got = out.download(np.float32, Q.shape)
        err = float(np.abs(got - want).max())
        assert err <= 2e-5, (qh, kvh, hd, ql, kl, err)
        done += 1


def _ids_equal_or_tie(got, want, gaps, scale):
    diff = np.flatnonzero(np.asarray(got) != np.asarray(want))
    return diff.size == 0 or gaps[int(diff[0])] <= _tie_bound(scale[int(diff[0])])


def test_random_model_configurations_through_every_host_mode(dev, orc):
    # small decoders of random shape (head_dim 16-128, 1-32 heads, FFN 64-5632, vocabulary 50-5000, 1-3 layers, either
    # RoPE layout, with and without biases, 1-5 sequences with prompts of 1-40 tokens) in the three host modes: greedy
    # decode of every prompt, then the packed prefill of all prompts (where the head size has one) with logits inside the
    # float bar and the batched decode from its cache -- ids equal to the oracle's, or parting at a pick inside the tie bound
    rng = np.random.default_rng(105)
    pick = lambda c: c[int(rng.integers(0, len(c)))]
    orc.set_threads(16)
    done = 0
    while done < 24:
        hd, kvh, g = pick([16, 32, 64, 128]), pick([1, 2, 4]), pick([1, 2, 4, 8])
        qh = kvh * g
        if qh * hd > 2048:
            continue
        cfg = dict(n_layers=pick([1, 2, 3]), d_model=qh * hd, q_heads=qh, kv_heads=kvh, head_dim=hd,
                   ffn=pick([64, 256, 384, 1000, 1536, 2048, 5632]), vocab=pick([50, 300, 1000, 5000]), rms_eps=1e-5,
                   rope_base=pick([10000.0, 1e6]), rope_scale=1.0, rope_layout=pick([0, 1]), qkv_bias=bool(pick([0, 1])))
        W = syn.make_weights(cfg, seed=int(rng.integers(0, 1000)), std=0.08, emb_std=1.0)
        S, B, n_gen = 80, pick([1, 2, 3, 5]), 5
        prompts = [rng.integers(0, cfg["vocab"], size=pick([1, 2, 7, 33, 40])).tolist() for _ in range(B)]
        lens = np.array([len(p) for p in prompts], dtype=np.uint32)
        om = orc.Model(dict(cfg), W)
        om.alloc_kv(S, B)
        want = [_oracle_greedy_with_logits(orc, om, s, p, n_gen) for s, p in enumerate(prompts)]
        om2 = orc.Model(dict(cfg), W)
        om2.alloc_kv(S, B)
        packed = hd in (64, 128)
        if packed:
            rows = om2.prefill_forward(list(range(B)), prompts)
            wl = [om2.logits(rows[e]) for e in np.cumsum(lens) - 1]
            firsts = [int(orc.greedy_topk1(l)) for l in wl]
            cont = [_oracle_greedy_with_logits(orc, om2, s, [firsts[s]], n_gen, start_pos=int(lens[s])) for s in range(B)]
        for mode in (0, 1, 2):
            dm = syn.DeviceModel(dev.ctx, cfg, W, max_seq_len=S, max_sequences=B)
            dm.set_mode(mode)
            for s, p in enumerate(prompts):
                got, _ = dm.decode_greedy(s, p, n_gen)
                assert _ids_equal_or_tie(got[len(p):], want[s][0][len(p):], want[s][1], want[s][2]), (cfg, mode, s)
            dm.close()
            if not packed:
                continue
            dm = syn.DeviceModel(dev.ctx, cfg, W, max_seq_len=S, max_sequences=B)
            dm.set_mode(mode)
            _, log = dm.forward_prefill(list(range(B)), prompts)
            for s in range(B):
                assert float(np.abs(log[s] - wl[s]).max()) <= 1e-3 * np.abs(wl[s]).max() + 1e-4, (cfg, mode, s)
            ids, _ = dm.decode_batch_greedy(np.arange(B), lens, firsts, n_gen)
            for s in range(B):
                assert _ids_equal_or_tie(ids[s], cont[s][0][1:], cont[s][1], cont[s][2]), (cfg, mode, s)
            dm.close()
        done += 1


def test_block_select_at_random_geometries(dev, orc):
    # contexts of 1-3000 tokens, windows of 1-1024, blocks of 1-100 tokens, 1-64 listed blocks, both old-V formats:
    # the listed block ids are the reference order's bit for bit, the output inside the float bar
    rng = np.random.default_rng(106)
    pick = lambda c: c[int(rng.integers(0, len(c)))]
    done = 0
    while done < 60:
        hd, kvh, g = pick([64, 128]), pick([1, 2, 4, 8]), pick([1, 2, 4, 8])
        qh = kvh * g
        L = pick([1, 2, 5, 17, 64, 65, 100, 300, 777, 1025, 2100, 3000])
        W, bs, top = pick([1, 2, 4, 16, 32, 100, 512, 1024]), pick([1, 2, 4, 16, 32, 48, 64, 100]), pick([1, 2, 3, 8, 17, 64])
        if qh * L * hd > 3e7:
            continue
        r = _block_select_case(dev, orc, qh, kvh, hd, L, W, bs, top, seed=int(rng.integers(0, 1000)), backing=pick([2, 2, 3]))
        case = (qh, kvh, hd, L, W, bs, top)
        assert np.array_equal(r["cnt"], r["wcnt"]), case
        assert np.array_equal(r["sel"], r["wsel"]), case
        close(r["got"], r["want"])
        done += 1


def test_scheduler_random_request_streams(dev, orc):
    # small decoders of random shape behind the scheduler: 1-4 slots, 3-10 requests with prompts of 1-31 tokens and 1-9
    # new tokens arriving over the first dozen ticks, one in seven cancelled two ticks after its arrival, any host mode.
    # Every request completes (or stays cancelled) and its tokens are the oracle's for that request alone -- the prompt
    # through the oracle's packed prefill where the scheduler packs prompts -- or part at a pick inside the tie bound.
    rng = np.random.default_rng(107)
    pick = lambda c: c[int(rng.integers(0, len(c)))]
    orc.set_threads(16)
    for _ in range(40):
        hd, kvh, g = pick([16, 64, 128]), pick([1, 2]), pick([1, 2, 4])
        qh = kvh * g
        cfg = dict(n_layers=pick([1, 2]), d_model=qh * hd, q_heads=qh, kv_heads=kvh, head_dim=hd, ffn=pick([128, 512, 1000]),
                   vocab=pick([60, 300, 2000]), rms_eps=1e-5, rope_base=10000.0, rope_scale=1.0, rope_layout=pick([0, 1]),
                   qkv_bias=bool(pick([0, 1])))
        W = syn.make_weights(cfg, seed=int(rng.integers(0, 1000)), std=0.08, emb_std=1.0)
        S, slots, mode = 64, pick([1, 2, 3, 4]), pick([0, 1, 2])
        dm = syn.DeviceModel(dev.ctx, cfg, W, max_seq_len=S, max_sequences=slots)
        dm.set_mode(mode)
        s = sch.Scheduler.for_model(dm)
        specs = [(rng.integers(0, cfg["vocab"], size=pick([1, 2, 9, 20, 31])).tolist(), pick([1, 2, 5, 9]), int(rng.integers(0, 12)),
                  bool(rng.random() < 0.15)) for _ in range(pick([3, 6, 10]))]
        rids, cancel_at, tick = {}, {}, 0
        pending = sorted(range(len(specs)), key=lambda i: specs[i][2])
        while pending or s.active():
            while pending and specs[pending[0]][2] <= tick and s.available_slots():
                i = pending.pop(0)
                rids[i] = s.submit(specs[i][0], max_tokens=specs[i][1])
                if specs[i][3]:
                    cancel_at[i] = tick + 2
            for i in [i for i, t in cancel_at.items() if t == tick]:
                s.cancel(rids[i])
                del cancel_at[i]
            s.tick()
            tick += 1
            assert tick < 500
        for i, (prompt, gen, _, _) in enumerate(specs):
            om = orc.Model(dict(cfg), W)
            om.alloc_kv(S, 1)
            if hd in (64, 128):
                hidden = om.prefill_forward([0], [prompt])[-1]
                want, gaps, scale = _oracle_greedy_with_logits(orc, om, 0, [], gen, start_pos=len(prompt), hidden=hidden)
            else:
                want, gaps, scale = _oracle_greedy_with_logits(orc, om, 0, prompt, gen)
                want = want[len(prompt):]
            got, state = s.generated(rids[i]), s.state(rids[i])
            assert state in ("complete", "cancelled"), (cfg, i, state, s.error(rids[i]))
            assert state == "cancelled" or len(got) == gen, (cfg, i, got)
            assert _ids_equal_or_tie(got, want[:len(got)], gaps, scale), (cfg, mode, i, got, want)
        assert s.available_slots() == slots
        s.close()
        dm.close()
