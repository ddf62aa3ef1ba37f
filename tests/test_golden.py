"""The reference's own literal test vectors (tests/golden/reference_literals.json) against the CPU oracle and
the host layer (no GPU needed), and against the HIP library through the C ABI (marked gpu).  Where the
reference's tests build inputs from a formula and recompute the expectation, the fixture holds the formula's
parameters and the expectation is recomputed here in float64, independently of the oracle."""
import ctypes as C
import importlib
import json
import os

import numpy as np
import pytest

m40 = importlib.import_module("m40-llm_amd")

with open(os.path.join(os.path.dirname(__file__), "golden", "reference_literals.json")) as _f:
    G = json.load(_f)


def _f16bits(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32).astype(np.float16).view(np.uint16))


def _logits(entry):
    return np.array([np.nan if v == "nan" else v for v in entry["logits"]], dtype=np.float32)


def _ramp(n, spec):
    """i*step + offset (or base + i*step), evaluated in f32 like the reference's `(i as f32) * step + offset`"""
    i = np.arange(n, dtype=np.float32)
    if "offset" in spec:
        return (i * np.float32(spec["step"]) + np.float32(spec["offset"])).astype(np.float32)
    return (np.float32(spec["base"]) + i * np.float32(spec["step"])).astype(np.float32)


def _q80_rows(g):
    sc, qn = g["scale"], g["quant"]
    for row in range(g["rows"]):
        d = np.array([sc["base"] + sc["per_row"] * row + sc["per_block"] * b for b in range(g["blocks_per_row"])],
                     dtype=np.float32).astype(np.float16)
        qs = np.array([[((qn["row_mul"] * row + qn["block_mul"] * b + i) % qn["modulus"]) + qn["offset"]
                        for i in range(32)] for b in range(g["blocks_per_row"])], dtype=np.int8)
        blob = np.zeros((g["blocks_per_row"], 34), dtype=np.uint8)
        blob[:, :2] = d.view(np.uint8).reshape(-1, 2)
        blob[:, 2:] = qs.view(np.uint8)
        yield blob, (d.astype(np.float64)[:, None] * qs.astype(np.float64)).reshape(-1)


def _config1_case(L):
    g = G["attention_gqa_config1"]
    kv_dim = g["kv_heads"] * g["head_dim"]
    t = np.arange(L)[:, None]; i = np.arange(kv_dim)[None, :]
    k = (t * kv_dim + i).astype(np.float32) * np.float32(g["k"]["scale"]) + np.float32(g["k"]["offset"])
    v = (t * kv_dim + (kv_dim - 1 - i)).astype(np.float32) * np.float32(g["v"]["scale"]) + np.float32(g["v"]["offset"])
    q = np.arange(g["q_heads"] * g["head_dim"], dtype=np.float32) * np.float32(g["q"]["scale"]) + np.float32(g["q"]["offset"])
    K = k.astype(np.float16).astype(np.float64).reshape(L, g["kv_heads"], g["head_dim"])
    V = v.astype(np.float16).astype(np.float64).reshape(L, g["kv_heads"], g["head_dim"])
    want = np.zeros((g["q_heads"], g["head_dim"]))
    grp = g["q_heads"] // g["kv_heads"]
    for h in range(g["q_heads"]):
        s = K[:, h // grp] @ q.reshape(g["q_heads"], -1)[h].astype(np.float64) / np.sqrt(g["head_dim"])
        p = np.exp(s - s.max()); p /= p.sum()
        want[h] = p @ V[:, h // grp]
    return k, v, q, want.reshape(-1)


# ---------------------------------------------------------------- oracle and host layer (CPU)
def test_oracle_kv_layout_literals(orc):
    g = G["kv_layout"]; L = orc.lib()
    dims = (g["max_seq_len"], g["num_heads"], g["head_dim"])
    assert L.orc_kv_elems_per_token(g["num_heads"], g["head_dim"]) == g["elems_per_token"]
    for e in g["base_offset_elems"]:
        assert L.orc_kv_base(*dims, e["seq"], e["token"]) == e["want"]
    for e in g["index_elems"]:
        assert L.orc_kv_index(*dims, e["seq"], e["token"], e["head"], e["dim"]) == e["want"]


def test_oracle_gemm_literals(orc):
    for e in G["gemm_rowmajor"]:
        a = np.array(e["a"], dtype=np.float32); b = np.array(e["b"], dtype=np.float32)
        m, n, k = e["m"], e["n"], e["k"]
        assert np.array_equal(orc.gemm("f16xf16_rowmajor", _f16bits(a), _f16bits(b), m, n, k), e["c"])
        assert np.array_equal(orc.gemm("f32xf16_rowmajor", a, _f16bits(b), m, n, k), e["c"])
        assert np.array_equal(orc.gemm("f32xf16_gguf", a, _f16bits(b.T), m, n, k), e["c"])


def test_oracle_q80_blocks(orc):
    for blob, want in _q80_rows(G["q80_blocks"]):
        assert np.array_equal(orc.q80_to_f32(blob, want.size).astype(np.float64), want)


def test_oracle_compressed_cache_bytes(orc):
    g = G["compressed_cache_bytes"]
    c = orc.CompressedKV(g["max_seq_len"], g["max_batch_size"], g["kv_heads"], g["head_dim"], g["recent_window"], g["block_size"])
    assert c.bytes() == (g["k_bytes"], g["v_q4_bytes"], g["v_scale_bytes"])


def test_oracle_and_host_sampler_greedy_literals(orc):
    H = m40.host()
    for e in G["greedy"]:
        lg = _logits(e)
        if e["top_k"] == 0:
            assert orc.sample_greedy(lg) == e["want"]
            s = H.m40host_sampler_create(1.0, -1, 0.0, 42)
            assert H.m40host_sampler_sample_greedy(s, lg.ctypes.data_as(C.c_void_p), lg.size) == e["want"]
        else:
            assert orc.greedy_topk1(lg) == e["want"]
            s = H.m40host_sampler_create(1.0, e["top_k"], 0.0, 42)
            assert H.m40host_sampler_sample(s, lg.ctypes.data_as(C.c_void_p), lg.size) == e["want"]
        H.m40host_sampler_destroy(s)


def test_oracle_kv_append_cast(orc):
    g = G["kv_append_fixtures"]
    for elems in g["elems"]:
        for pair in g["pairs"]:
            for spec in (pair["k"], pair["v"]):
                x = _ramp(elems, spec)
                assert np.array_equal(orc.f32_to_f16_bits(x), x.astype(np.float16).view(np.uint16))


def test_oracle_attention_config1(orc):
    g = G["attention_gqa_config1"]
    for L in g["seq_lens"]:
        k, v, q, want = _config1_case(L)
        K = _f16bits(k).reshape(1, L, g["kv_heads"], g["head_dim"]); V = _f16bits(v).reshape(K.shape)
        got = orc.attention(K, V, L, g["kv_heads"], g["head_dim"], 0, q, g["q_heads"], L)
        assert np.allclose(got, want, rtol=1e-4, atol=1e-5)


def test_oracle_rms_norm_and_rope(orc):
    g = G["rms_norm"]
    rows, dim, eps = g["rows"], g["dim"], g["eps"]
    x = _ramp(rows * dim, g["plain_x"]).reshape(rows, dim)
    x64 = x.astype(np.float64)
    assert np.allclose(orc.rms_norm(x, eps), x64 / np.sqrt((x64 ** 2).mean(1, keepdims=True) + eps), rtol=1e-6, atol=1e-7)
    x = _ramp(rows * dim, g["weighted_x"]).reshape(rows, dim); w = _ramp(dim, g["weight"])
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt((x64 ** 2).mean(1, keepdims=True) + eps) * w.astype(np.float64)
    assert np.allclose(orc.rms_norm(x, eps, w, 1), want, rtol=1e-6, atol=1e-7)
    g = G["rope_adjacent"]
    for case in g["cases"]:
        x = _ramp(case["rows"] * g["heads"] * g["head_dim"], g["x"]).reshape(case["rows"], -1)
        assert np.allclose(orc.rope(x, g["heads"], g["head_dim"], case["past_len"], g["base"], g["scale"], 0),
                           _rope_adjacent_f64(x, g, case["past_len"]), rtol=1e-5, atol=1e-6)


def _rope_adjacent_f64(x, g, past):
    rows = x.shape[0]; hd = g["head_dim"]
    t = x.astype(np.float64).reshape(rows, g["heads"], hd // 2, 2)
    pos = (past + np.arange(rows))[:, None, None] * g["scale"]
    th = pos * g["base"] ** (-2.0 * np.arange(hd // 2) / hd)[None, None, :]
    out = np.empty_like(t)
    out[..., 0] = t[..., 0] * np.cos(th) - t[..., 1] * np.sin(th)
    out[..., 1] = t[..., 0] * np.sin(th) + t[..., 1] * np.cos(th)
    return out.reshape(rows, -1)


def test_host_batch_plan_and_pool_literals():
    H = m40.host()
    g = G["decode_batch_plan"]
    code = {"active": 0, "completed": 1, "cancelled": 2}
    reqs = g["requests"]
    rid = np.array([r["request_id"] for r in reqs], dtype=np.uint64)
    sid = np.array([r["sequence_id"] for r in reqs], dtype=np.uint32)
    kvl = np.array([r["kv_len"] for r in reqs], dtype=np.uint32)
    st = np.array([code[r["state"]] for r in reqs], dtype=np.uint32)
    vp = lambda a: a.ctypes.data_as(C.c_void_p)
    p = H.m40host_batch_plan_from_requests(vp(rid), vp(sid), vp(kvl), vp(st), len(reqs))
    n = len(g["sequence_ids"])
    assert p and H.m40host_batch_plan_size(p) == n
    ids = np.zeros(n, dtype=np.uint32); lens = np.zeros(n, dtype=np.uint32)
    H.m40host_batch_plan_sequence_ids(p, vp(ids)); H.m40host_batch_plan_sequence_lens(p, vp(lens))
    assert list(ids) == g["sequence_ids"] and list(lens) == g["sequence_lens"]
    assert H.m40host_batch_plan_total_q_tokens(p) == g["total_q_tokens"]
    assert H.m40host_batch_plan_total_kv_tokens(p) == g["total_kv_tokens"]
    for r, want in g["batch_index_for_request"].items():
        assert H.m40host_batch_plan_index_for_request(p, int(r)) == want
    o = g["output_offset_f32"]
    assert H.m40host_batch_plan_output_offset_f32(p, o["request_id"], o["q_heads"], o["head_dim"]) == o["want"]
    H.m40host_batch_plan_destroy(p)

    g = G["sequence_pool"]
    pool = H.m40host_pool_create(g["capacity"])
    leases = [H.m40host_pool_try_lease(pool) for _ in g["leases"]]
    assert [H.m40host_lease_sequence_id(l) for l in leases] == g["leases"]
    assert (H.m40host_pool_try_lease(pool) is None) == g["third_is_none"]
    H.m40host_lease_release(leases[0])
    nxt = H.m40host_pool_try_lease(pool)
    assert H.m40host_lease_sequence_id(nxt) == g["after_dropping_first_next"]
    H.m40host_lease_release(nxt); H.m40host_lease_release(leases[1])
    H.m40host_pool_destroy(pool)


# ---------------------------------------------------------------- HIP library through the C ABI
@pytest.fixture(scope="module")
def dev():
    from gpu_common import Dev
    d = Dev()
    yield d
    d.sync()


@pytest.mark.gpu
def test_gpu_gemm_literals(dev):
    for e in G["gemm_rowmajor"]:
        a = np.array(e["a"], dtype=np.float32); b = np.array(e["b"], dtype=np.float32)
        m, n, k = e["m"], e["n"], e["k"]
        dC = dev.zeros(m * n * 4)
        for sym, A, B in (("m40llm_gemm_f16xf16_f32", _f16bits(a), _f16bits(b)),
                          ("m40llm_gemm_f32xf16_f32", a, _f16bits(b)),
                          ("m40llm_gemm_f32xf16_gguf_f32", a, _f16bits(b.T))):
            dA, dB = dev.up(A), dev.up(B)
            dev.call(sym, dA.ptr, dB.ptr, dC.ptr, m, n, k)
            assert np.array_equal(dC.download(np.float32, (m, n)), e["c"]), sym


@pytest.mark.gpu
def test_gpu_q80_blocks(dev):
    for blob, want in _q80_rows(G["q80_blocks"]):
        din, dout = dev.up(blob), dev.zeros(want.size * 4)
        dev.call("m40llm_q80_to_f32", din.ptr, dout.ptr, want.size)
        assert np.array_equal(dout.download(np.float32, (want.size,)).astype(np.float64), want)


@pytest.mark.gpu
def test_gpu_greedy_literals(dev):
    for e in G["greedy"]:
        lg = _logits(e)
        dx, di = dev.up(lg), dev.zeros(4)
        dev.call("m40llm_ext_argmax_f32_async", dx.ptr, 1, lg.size, di.ptr, None)
        dev.sync()
        assert int(di.download(np.uint32, (1,))[0]) == e["want"]


@pytest.mark.gpu
def test_gpu_kv_layout_and_append_cast(dev):
    g = G["kv_layout"]
    kv = m40.KVCache(dev.ctx, g["max_seq_len"], g["max_batch_size"], g["num_heads"], g["head_dim"])
    elems = g["elems_per_token"]
    # token t of sequence 1 holds the values base(1, t) + i, so the element at the cited flat index is its own index
    for t in range(3):
        k = (g["base_offset_elems"][2]["want"] + t * elems + np.arange(elems)).astype(np.float32)
        dk, dv = dev.up(k), dev.up(-k)
        dev.call("m40llm_kvcache_append_token_f32", kv.h, 1, dk.ptr, dv.ptr)
    raw = np.zeros(g["max_seq_len"] * g["max_batch_size"] * elems, dtype=np.uint16)
    for s in range(g["max_batch_size"]):
        for t in range(g["max_seq_len"]):
            kk, _ = kv.read_token(s, t)
            base = (s * g["max_seq_len"] + t) * elems
            raw[base:base + elems] = kk.reshape(-1)
    for e in g["index_elems"]:
        assert raw.view(np.float16)[e["want"]] == e["want"]
    assert not raw[:g["base_offset_elems"][2]["want"]].any()

    g = G["kv_append_fixtures"]
    for elems in g["elems"]:
        kv = m40.KVCache(dev.ctx, 4, 1, 1, elems)
        for t, pair in enumerate(g["pairs"]):
            k, v = _ramp(elems, pair["k"]), _ramp(elems, pair["v"])
            dk, dv = dev.up(k), dev.up(v)
            dev.call("m40llm_kvcache_append_token_f32", kv.h, 0, dk.ptr, dv.ptr)
            gk, gv = kv.read_token(0, t)
            assert np.array_equal(gk.reshape(-1), k.astype(np.float16).view(np.uint16))
            assert np.array_equal(gv.reshape(-1), v.astype(np.float16).view(np.uint16))


@pytest.mark.gpu
def test_gpu_attention_config1(dev):
    from gpu_common import close
    g = G["attention_gqa_config1"]
    for L in g["seq_lens"]:
        k, v, q, want = _config1_case(L)
        kv = m40.KVCache(dev.ctx, L, 1, g["kv_heads"], g["head_dim"])
        dev.fill_dense(kv, 0, _f16bits(k).reshape(L, g["kv_heads"], g["head_dim"]),
                       _f16bits(v).reshape(L, g["kv_heads"], g["head_dim"]))
        close(dev.attention(kv, 0, q, g["q_heads"], L), want)


@pytest.mark.gpu
def test_gpu_rms_norm_and_rope(dev):
    from gpu_common import close
    g = G["rms_norm"]
    rows, dim, eps = g["rows"], g["dim"], g["eps"]
    x = _ramp(rows * dim, g["plain_x"]).reshape(rows, dim)
    x64 = x.astype(np.float64)
    dx, dy = dev.up(x), dev.zeros(x.nbytes)
    dev.call("m40llm_rms_norm_f32", dx.ptr, dy.ptr, rows, dim, eps)
    close(dy.download(np.float32, x.shape), x64 / np.sqrt((x64 ** 2).mean(1, keepdims=True) + eps), 1e-5, 1e-6)
    g = G["rope_adjacent"]
    for case in g["cases"]:
        x = _ramp(case["rows"] * g["heads"] * g["head_dim"], g["x"]).reshape(case["rows"], -1)
        dx = dev.up(x)
        dev.call("m40llm_rope_f32_inplace_layout_async", dx.ptr, case["rows"], g["heads"], g["head_dim"],
                 case["past_len"], g["base"], g["scale"], 0)
        dev.sync()
        close(dx.download(np.float32, x.shape), _rope_adjacent_f64(x, g, case["past_len"]), 1e-5, 1e-6)
