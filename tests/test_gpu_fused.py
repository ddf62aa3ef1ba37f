"""Fused batch-1 decode entry points: each one must equal, bit for bit, the chain of reference-named
entry points it stands for (src/infer/forward.rs:304-662 issues them one by one), and sit within the
float tolerance of the CPU oracle."""
import ctypes as C

import numpy as np
import pytest

from gpu_common import Dev, close, f16bits, m40

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    d = Dev()
    yield d
    d.ctx.close()


def _gemv(dev, dA, dB, N, K):
    dC = dev.zeros(N * 4)
    dev.call("m40llm_ext_gemm_f32xf16_gguf_f32_async", dA.ptr, dB.ptr, dC.ptr, 1, N, K, 1)
    return dC


@pytest.mark.parametrize("qh,kvh,hd,d_model,layout,bias,base", [
    (32, 4, 64, 2048, 0, False, 1e4),     # TinyLlama-1.1B layer
    (16, 2, 128, 2048, 1, True, 1e6),     # Qwen2.5-3B layer: NeoX pairs, QKV bias
    (4, 2, 32, 256, 0, True, 1e4),
])
def test_norm_qkv_rope_append_equals_call_sequence(dev, orc, qh, kvh, hd, d_model, layout, bias, base):
    rng = np.random.default_rng(qh * 131 + hd)
    K = d_model
    x = rng.standard_normal(K).astype(np.float32)
    nw = (1 + 0.1 * rng.standard_normal(K)).astype(np.float32)
    wq = f16bits(rng.standard_normal((qh * hd, K)) * 0.03)
    wk = f16bits(rng.standard_normal((kvh * hd, K)) * 0.03)
    wv = f16bits(rng.standard_normal((kvh * hd, K)) * 0.03)
    bq = rng.standard_normal(qh * hd).astype(np.float32) * 0.1
    bk = rng.standard_normal(kvh * hd).astype(np.float32) * 0.1
    bv = rng.standard_normal(kvh * hd).astype(np.float32) * 0.1
    dx, dnw, dwq, dwk, dwv = dev.up(x), dev.up(nw), dev.up(wq), dev.up(wk), dev.up(wv)
    dbq, dbk, dbv = dev.up(bq), dev.up(bk), dev.up(bv)
    eps = 1e-5
    for position in (0, 5, 61):
        kv_f = m40.KVCache(dev.ctx, 64, 2, kvh, hd)
        kv_u = m40.KVCache(dev.ctx, 64, 2, kvh, hd)
        # fused, position from the device
        dpos = dev.up(np.array([position], dtype=np.uint32))
        dq_f = dev.zeros(qh * hd * 4)
        dev.call("m40llm_ext_fused_norm_qkv_rope_append_async", kv_f.h, 1, dx.ptr, dnw.ptr, 1, eps, dwq.ptr, dwk.ptr,
                 dwv.ptr, dbq.ptr if bias else None, dbk.ptr if bias else None, dbv.ptr if bias else None, K, qh, 12345,
                 dpos.ptr, base, 1.0, layout, dq_f.ptr)
        # reference call sequence
        dxn = dev.zeros(K * 4)
        dev.call("m40llm_rms_norm_f32_weighted_async", dx.ptr, dnw.ptr, dxn.ptr, 1, K, eps, 1)
        dq_u = _gemv(dev, dxn, dwq, qh * hd, K)
        dk_u = _gemv(dev, dxn, dwk, kvh * hd, K)
        dv_u = _gemv(dev, dxn, dwv, kvh * hd, K)
        if bias:
            dev.call("m40llm_residual_add_f32_async", dq_u.ptr, dbq.ptr, dq_u.ptr, qh * hd)
            dev.call("m40llm_residual_add_f32_async", dk_u.ptr, dbk.ptr, dk_u.ptr, kvh * hd)
            dev.call("m40llm_residual_add_f32_async", dv_u.ptr, dbv.ptr, dv_u.ptr, kvh * hd)
        dev.call("m40llm_rope_f32_inplace_layout_async", dq_u.ptr, 1, qh, hd, position, base, 1.0, layout)
        dev.call("m40llm_kvcache_append_token_f32_rope_k_at_layout_async", kv_u.h, 1, dk_u.ptr, dv_u.ptr, position,
                 position, base, 1.0, layout)
        dev.sync()
        q_f = dq_f.download(np.float32, (qh * hd,)); q_u = dq_u.download(np.float32, (qh * hd,))
        assert np.array_equal(q_f.view(np.uint32), q_u.view(np.uint32))
        kf, vf = kv_f.read_token(1, position); ku, vu = kv_u.read_token(1, position)
        for name, a, b in (("K", kf, ku), ("V", vf, vu)):
            bad = np.flatnonzero(a != b)
            assert bad.size == 0, (name, position, bad.size, bad[:8], a[bad[:8]], b[bad[:8]])
        # oracle
        xn = orc.rms_norm(x[None], eps, nw, 1)
        q_o = orc.gemm("f32xf16_gguf", xn, wq, 1, qh * hd, K) + (bq if bias else 0)
        q_o = orc.rope(q_o.astype(np.float32), qh, hd, position, base, 1.0, layout)
        close(q_f, q_o[0])
        k_o = orc.gemm("f32xf16_gguf", xn, wk, 1, kvh * hd, K) + (bk if bias else 0)
        k_o = orc.rope(k_o.astype(np.float32), kvh, hd, position, base, 1.0, layout)
        close(kf.view(np.float16).astype(np.float32), k_o[0], 2e-3, 1e-3)   # f16 storage rounding
        kv_f.destroy(); kv_u.destroy()


@pytest.mark.parametrize("N,K", [(2048, 2048), (2048, 5632), (2048, 11008), (8192, 2048), (300, 4096), (33, 64)])
def test_gemv_residual_equals_call_sequence(dev, orc, N, K):
    rng = np.random.default_rng(N + K)
    a = rng.standard_normal(K).astype(np.float32)
    r = rng.standard_normal(N).astype(np.float32)
    W = f16bits(rng.standard_normal((N, K)) * 0.02)
    da, dr, dW = dev.up(a), dev.up(r), dev.up(W)
    out_f = dev.zeros(N * 4)
    dev.call("m40llm_ext_gemv_residual_f32xf16_async", da.ptr, dW.ptr, dr.ptr, out_f.ptr, N, K)
    y = _gemv(dev, da, dW, N, K)
    out_u = dev.zeros(N * 4)
    dev.call("m40llm_residual_add_f32_async", dr.ptr, y.ptr, out_u.ptr, N)
    dev.sync()
    got = out_f.download(np.float32, (N,))
    assert np.array_equal(got.view(np.uint32), out_u.download(np.float32, (N,)).view(np.uint32))
    want = r + orc.gemm("f32xf16_gguf", a[None], W, 1, N, K)[0]
    close(got, want)
    # in place (residual aliases out), and without a residual
    dev.call("m40llm_ext_gemv_residual_f32xf16_async", da.ptr, dW.ptr, dr.ptr, dr.ptr, N, K)
    dev.call("m40llm_ext_gemv_residual_f32xf16_async", da.ptr, dW.ptr, None, out_f.ptr, N, K)
    dev.sync()
    assert np.array_equal(dr.download(np.float32, (N,)), got)
    assert np.array_equal(out_f.download(np.float32, (N,)), y.download(np.float32, (N,)))


@pytest.mark.parametrize("F,K", [(5632, 2048), (11008, 2048), (130, 256)])
def test_norm_gate_up_swiglu_equals_call_sequence(dev, orc, F, K):
    rng = np.random.default_rng(F)
    x = rng.standard_normal(K).astype(np.float32) * 3
    nw16 = f16bits(1 + 0.1 * rng.standard_normal(K))
    wg = f16bits(rng.standard_normal((F, K)) * 0.03); wu = f16bits(rng.standard_normal((F, K)) * 0.03)
    dx, dnw, dwg, dwu = dev.up(x), dev.up(nw16), dev.up(wg), dev.up(wu)
    hid_f = dev.zeros(F * 4)
    dev.call("m40llm_ext_fused_norm_gate_up_swiglu_async", dx.ptr, dnw.ptr, 0, 1e-6, dwg.ptr, dwu.ptr, hid_f.ptr, F, K)
    dxn = dev.zeros(K * 4)
    dev.call("m40llm_rms_norm_f32_weighted_async", dx.ptr, dnw.ptr, dxn.ptr, 1, K, 1e-6, 0)
    g = _gemv(dev, dxn, dwg, F, K); u = _gemv(dev, dxn, dwu, F, K)
    hid_u = dev.zeros(F * 4)
    dev.call("m40llm_swiglu_f32_async", g.ptr, u.ptr, hid_u.ptr, F)
    dev.sync()
    got = hid_f.download(np.float32, (F,))
    assert np.array_equal(got.view(np.uint32), hid_u.download(np.float32, (F,)).view(np.uint32))
    xn = orc.rms_norm(x[None], 1e-6, nw16, 0)
    want = orc.swiglu(orc.gemm("f32xf16_gguf", xn, wg, 1, F, K), orc.gemm("f32xf16_gguf", xn, wu, 1, F, K))[0]
    close(got, want)


@pytest.mark.parametrize("V,K", [(32000, 2048), (151936, 2048), (1000, 256), (5, 64)])
def test_lm_head_top2_and_greedy_step(dev, orc, V, K):
    rng = np.random.default_rng(V)
    x = rng.standard_normal(K).astype(np.float32)
    nw = (1 + 0.1 * rng.standard_normal(K)).astype(np.float32)
    W = f16bits(rng.standard_normal((V, K)) * 0.02)
    table = f16bits(rng.standard_normal((V, K)))
    if V >= 1000:
        W[V - 3] = W[17]                     # exact tie between two columns: the lower index must win
        x_big = np.sign(W[17].view(np.float16).astype(np.float32))
        x = (x + 4 * x_big).astype(np.float32)   # ... and make that pair the maximum
    dx, dnw, dW, dT = dev.up(x), dev.up(nw), dev.up(W), dev.up(table)
    cap = 1 << 16
    top2 = dev.zeros(3 * cap * 4)
    logits = dev.zeros(V * 4)
    nblk = C.c_uint32(0)
    dev.call("m40llm_ext_fused_norm_gemv_f32xf16_async", dx.ptr, dnw.ptr, 1, 1e-5, dW.ptr, logits.ptr, V, K, top2.ptr,
             cap, C.byref(nblk))
    # unfused twin
    dxn = dev.zeros(K * 4)
    dev.call("m40llm_rms_norm_f32_weighted_async", dx.ptr, dnw.ptr, dxn.ptr, 1, K, 1e-5, 1)
    lg_u = _gemv(dev, dxn, dW, V, K)
    dev.sync()
    lg = logits.download(np.float32, (V,))
    assert np.array_equal(lg.view(np.uint32), lg_u.download(np.float32, (V,)).view(np.uint32))
    close(lg, orc.gemm("f32xf16_gguf", orc.rms_norm(x[None], 1e-5, nw, 1), W, 1, V, K)[0])
    assert 0 < nblk.value <= cap
    # greedy step from the candidates and from a plain scan; state = {position, step, token, capacity, ids, gaps}
    scap = 4
    want_tok = orc.sample_greedy(lg)
    assert want_tok == int(np.argmax(lg))
    srt = np.sort(lg)
    for use_top2 in (True, False):
        st = np.zeros(4 + 2 * scap, dtype=np.uint32); st[0] = 9; st[1] = 1; st[3] = scap
        dst = dev.up(st)
        xout = dev.zeros(K * 4)
        dev.call("m40llm_ext_greedy_step_async", logits.ptr, V, top2.ptr if use_top2 else None, cap,
                 nblk.value if use_top2 else 0, dst.ptr, dT.ptr, K, xout.ptr)
        dev.sync()
        got = dst.download(np.uint32, st.shape)
        assert got[0] == 10 and got[1] == 2 and got[3] == scap
        assert got[2] == want_tok and got[4 + 1] == want_tok
        gap = got[4 + scap + 1: 4 + scap + 2].view(np.float32)[0]
        assert gap == srt[-1] - srt[-2]
        assert np.array_equal(xout.download(np.float32, (K,)), table[want_tok].view(np.float16).astype(np.float32))
    if V >= 1000:
        assert want_tok == 17 and srt[-1] == srt[-2]
    # capacity check and argument validation
    assert dev.lib.m40llm_ext_fused_norm_gemv_f32xf16_async(dev.h, dx.ptr, dnw.ptr, 1, 1e-5, dW.ptr, logits.ptr, V, K,
                                                            top2.ptr, 0, None) == -5
    assert dev.lib.m40llm_ext_greedy_step_async(dev.h, None, V, None, 0, 0, dst.ptr, None, 0, None) == -1
