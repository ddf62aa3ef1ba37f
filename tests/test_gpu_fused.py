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
        close(kf.view(np.float16).astype(np.float32), k_o[0])   # f16 storage rounding: half a step, 2^-11 relative
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


# ------------------------------------------------------------------ row-batched fused entry points
def _rows_case(rng, rows, K):
    x = rng.standard_normal((rows, K)).astype(np.float32)
    if rows > 1:
        x[1] *= 1e-3            # rows of very different magnitude (per-row, per-step scaling of the f16 split)
    if rows > 2:
        x[2] *= 3e3
    return x


@pytest.mark.parametrize("rows", [1, 8, 13])
def test_batched_gemm_residual_and_norm_gate_up_vs_oracle(dev, orc, rows):
    rng = np.random.default_rng(rows)
    D, F = 512, 768
    x = _rows_case(rng, rows, D)
    nw = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    wg = f16bits(rng.standard_normal((F, D)) * 0.05); wu = f16bits(rng.standard_normal((F, D)) * 0.05)
    wd = f16bits(rng.standard_normal((D, F)) * 0.05)
    dx, dnw, dwg, dwu, dwd = dev.up(x), dev.up(nw), dev.up(wg), dev.up(wu), dev.up(wd)
    hid = dev.zeros(rows * F * 4)
    dev.call("m40llm_ext_batched_norm_gate_up_swiglu_async", dx.ptr, dnw.ptr, 1, 1e-5, dwg.ptr, dwu.ptr, hid.ptr, rows, F, D)
    out = dev.zeros(rows * D * 4)
    dev.call("m40llm_ext_batched_gemm_residual_f32xf16_async", hid.ptr, dwd.ptr, dx.ptr, out.ptr, rows, D, F)
    dev.sync()
    xn = orc.rms_norm(x, 1e-5, nw, 1)
    want_h = orc.swiglu(orc.gemm("f32xf16_gguf", xn, wg, rows, F, D), orc.gemm("f32xf16_gguf", xn, wu, rows, F, D))
    got_h = hid.download(np.float32, (rows, F))
    sc = np.abs(want_h).max(axis=1, keepdims=True)
    close(got_h / sc, want_h / sc)
    want = x + orc.gemm("f32xf16_gguf", want_h, wd, rows, D, F)
    got = out.download(np.float32, (rows, D))
    sc = np.abs(want).max(axis=1, keepdims=True)
    close(got / sc, want / sc)
    # argument checks: more than 16 rows, K not a multiple of 256
    dev.call("m40llm_ext_batched_gemm_residual_f32xf16_async", hid.ptr, dwd.ptr, dx.ptr, out.ptr, 17, D, F, expect=-6)
    dev.call("m40llm_ext_batched_gemm_residual_f32xf16_async", hid.ptr, dwd.ptr, dx.ptr, out.ptr, rows, D, F - 64, expect=-6)


@pytest.mark.parametrize("rows,F,V,norm_dtype", [(1, 1004, 1000, 1), (5, 2056, 4099, 0), (8, 5632, 20011, 1)])
def test_batched_projections_at_k2048_vs_oracle(dev, orc, rows, F, V, norm_dtype):
    # d_model 2048 with up to eight rows takes the persistent matrix-core kernel: gate/up + SwiGLU with column tails
    # (F not a multiple of 8), lm_head-style norm + product (V not a multiple of 16), and a wide residual product
    rng = np.random.default_rng(100 + rows)
    D = 2048
    x = _rows_case(rng, rows, D)
    nw = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    if norm_dtype == 0:
        nw = nw.astype(np.float16).astype(np.float32)
    dnw = dev.up(f16bits(nw) if norm_dtype == 0 else nw)
    wg = f16bits(rng.standard_normal((F, D)) * 0.03); wu = f16bits(rng.standard_normal((F, D)) * 0.03)
    dx, dwg, dwu = dev.up(x), dev.up(wg), dev.up(wu)
    hid = dev.zeros(rows * F * 4)
    dev.call("m40llm_ext_batched_norm_gate_up_swiglu_async", dx.ptr, dnw.ptr, norm_dtype, 1e-5, dwg.ptr, dwu.ptr, hid.ptr, rows, F, D)
    dev.sync()
    xn = orc.rms_norm(x, 1e-5, nw, 1)
    want_h = orc.swiglu(orc.gemm("f32xf16_gguf", xn, wg, rows, F, D), orc.gemm("f32xf16_gguf", xn, wu, rows, F, D))
    got_h = hid.download(np.float32, (rows, F))
    sc = np.abs(want_h).max(axis=1, keepdims=True)
    close(got_h / sc, want_h / sc)
    # norm + product (the lm_head call)
    wv = f16bits(rng.standard_normal((V, D)) * 0.03)
    dwv, logits = dev.up(wv), dev.zeros(rows * V * 4)
    dev.call("m40llm_ext_batched_norm_gemm_f32xf16_async", dx.ptr, dnw.ptr, norm_dtype, 1e-5, dwv.ptr, logits.ptr, rows, V, D)
    dev.sync()
    want = orc.gemm("f32xf16_gguf", xn, wv, rows, V, D)
    got = logits.download(np.float32, (rows, V))
    sc = np.abs(want).max(axis=1, keepdims=True)
    close(got / sc, want / sc)
    for r in range(rows):
        assert int(np.argmax(got[r])) == int(np.argmax(want[r]))
    # product + residual, in place, wider than the vector-ALU kernel takes (N > 8192)
    if V > 8192:
        res = rng.standard_normal((rows, V)).astype(np.float32)
        dres = dev.up(res)
        dev.call("m40llm_ext_batched_gemm_residual_f32xf16_async", dx.ptr, dwv.ptr, dres.ptr, dres.ptr, rows, V, D)
        dev.sync()
        want = res + orc.gemm("f32xf16_gguf", x, wv, rows, V, D)
        got = dres.download(np.float32, (rows, V))
        sc = np.abs(want).max(axis=1, keepdims=True)
        close(got / sc, want / sc)


@pytest.mark.parametrize("rows,N,K", [(8, 2048, 11008), (5, 512, 5632), (3, 1000, 2304), (1, 2048, 4096), (8, 40, 8192)])
def test_batched_down_projection_k_chunks_vs_oracle(dev, orc, rows, N, K):
    # down-projection shapes (K > 2048, K slices summed with the residual by the slice-adding launch, in place; column
    # tail; fewer column tiles than the chip has CUs)
    rng = np.random.default_rng(rows + K)
    a = _rows_case(rng, rows, K)
    w = f16bits(rng.standard_normal((N, K)) * 0.03)
    res = rng.standard_normal((rows, N)).astype(np.float32)
    da, dw, dres = dev.up(a), dev.up(w), dev.up(res)
    dev.call("m40llm_ext_batched_gemm_residual_f32xf16_async", da.ptr, dw.ptr, dres.ptr, dres.ptr, rows, N, K)
    dev.sync()
    want = res + orc.gemm("f32xf16_gguf", a, w, rows, N, K)
    got = dres.download(np.float32, (rows, N))
    sc = np.abs(want).max(axis=1, keepdims=True)
    close(got / sc, want / sc)
    # a second call with other inputs through the same scratch slices, no residual
    a2 = _rows_case(rng, rows, K)
    da2, out = dev.up(a2), dev.zeros(rows * N * 4)
    dev.call("m40llm_ext_batched_gemm_residual_f32xf16_async", da2.ptr, dw.ptr, None, out.ptr, rows, N, K)
    dev.sync()
    want = orc.gemm("f32xf16_gguf", a2, w, rows, N, K)
    got = out.download(np.float32, (rows, N))
    sc = np.abs(want).max(axis=1, keepdims=True)
    close(got / sc, want / sc)


@pytest.mark.parametrize("rows,N,K", [(8, 2048, 11008), (5, 2040, 5632), (1, 4096, 4096), (3, 1027, 4352), (6, 2048, 4128), (7, 8192, 14336),
                                      (8, 512, 8192), (9, 2048, 11008), (4, 2048, 2048)])
def test_batched_down_projection_onto_zero_vs_oracle(dev, orc, rows, N, K):
    """Gate + up with the clear on the side (d_model 2048: the persistent kernel clears; otherwise a fill launch), then
    the down projection whose two K halves are added into the cleared result (up to eight rows, K >= 4096, 64 to 512
    column tiles; column tails, k-step counts that do not divide by the waves; other shapes fall to the overwriting
    form), against the oracle; the same call twice gives the same bits."""
    rng = np.random.default_rng(rows * 31 + K)
    a = _rows_case(rng, rows, K)
    w = f16bits(rng.standard_normal((N, K)) * 0.03)
    res = rng.standard_normal((rows, N)).astype(np.float32)
    da, dw, dres = dev.up(a), dev.up(w), dev.up(res)
    out = dev.up(np.full((rows, N), 7.0, dtype=np.float32))
    # the clear rides on a gate + up call (its own result is not used here)
    D = 2048
    x = _rows_case(rng, rows, D)
    nw = np.ones(D, dtype=np.float32)
    wg = f16bits(rng.standard_normal((64, D)) * 0.03)
    dx, dnw, dwg, hid = dev.up(x), dev.up(nw), dev.up(wg), dev.zeros(rows * 64 * 4)
    def run():
        dev.call("m40llm_ext_batched_norm_gate_up_swiglu_clear_async", dx.ptr, dnw.ptr, 1, 1e-5, dwg.ptr, dwg.ptr, hid.ptr, rows,
                 64, D, out.ptr, rows * N)
        dev.call("m40llm_ext_batched_gemm_residual_onto_zero_f32xf16_async", da.ptr, dw.ptr, dres.ptr, out.ptr, rows, N, K)
        dev.sync()
        return out.download(np.float32, (rows, N))
    got = run()
    want = res + orc.gemm("f32xf16_gguf", a, w, rows, N, K)
    sc = np.abs(want).max(axis=1, keepdims=True)
    close(got / sc, want / sc)
    f64 = res.astype(np.float64) + a.astype(np.float64) @ w.view(np.float16).astype(np.float64).T
    close(got / sc, f64 / sc, 1e-5, 1e-6)
    for _ in range(3):
        assert np.array_equal(run(), got)
    # no residual
    dev.call("m40llm_ext_batched_norm_gate_up_swiglu_clear_async", dx.ptr, dnw.ptr, 1, 1e-5, dwg.ptr, dwg.ptr, hid.ptr, rows, 64, D,
             out.ptr, rows * N)
    dev.call("m40llm_ext_batched_gemm_residual_onto_zero_f32xf16_async", da.ptr, dw.ptr, None, out.ptr, rows, N, K)
    dev.sync()
    close(out.download(np.float32, (rows, N)) / sc, (f64 - res) / sc, 1e-5, 1e-6)


@pytest.mark.parametrize("qh,kvh,hd,layout,bias,rows", [
    (8, 2, 64, 0, False, 5), (4, 2, 128, 1, True, 8), (4, 1, 128, 1, True, 12),
    # d_model 2048 with up to eight rows: the persistent matrix-core kernel (adjacent and split-half pairs, with and without bias)
    (32, 4, 64, 0, False, 5), (16, 2, 128, 1, True, 8), (32, 8, 64, 1, True, 1), (16, 4, 128, 0, True, 3)])
def test_batched_norm_qkv_rope_append_vs_oracle(dev, orc, qh, kvh, hd, layout, bias, rows):
    rng = np.random.default_rng(qh + rows)
    D = qh * hd
    x = _rows_case(rng, rows, D)
    nw = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    wq = f16bits(rng.standard_normal((qh * hd, D)) * 0.05)
    wk = f16bits(rng.standard_normal((kvh * hd, D)) * 0.05)
    wv = f16bits(rng.standard_normal((kvh * hd, D)) * 0.05)
    bq = (rng.standard_normal(qh * hd) * 0.1).astype(np.float32)
    bk = (rng.standard_normal(kvh * hd) * 0.1).astype(np.float32)
    bv = (rng.standard_normal(kvh * hd) * 0.1).astype(np.float32)
    nseq, S = 16, 64
    kv = m40.KVCache(dev.ctx, S, nseq, kvh, hd)
    ids = rng.permutation(nseq)[:rows].astype(np.uint32)
    lens = rng.integers(0, S, size=rows).astype(np.uint32)
    dx, dnw, dwq, dwk, dwv = dev.up(x), dev.up(nw), dev.up(wq), dev.up(wk), dev.up(wv)
    dbq, dbk, dbv = dev.up(bq), dev.up(bk), dev.up(bv)
    dids, dlens = dev.up(ids), dev.up(lens)
    dq = dev.zeros(rows * qh * hd * 4)
    base = 1e6 if layout else 1e4
    dev.call("m40llm_ext_batched_norm_qkv_rope_append_async", kv.h, dids.ptr, dlens.ptr, rows, dx.ptr, dnw.ptr, 1, 1e-6,
             dwq.ptr, dwk.ptr, dwv.ptr, dbq.ptr if bias else None, dbk.ptr if bias else None, dbv.ptr if bias else None,
             D, qh, base, 1.0, layout, dq.ptr)
    dev.sync()
    got_q = dq.download(np.float32, (rows, qh * hd))
    xn = orc.rms_norm(x, 1e-6, nw, 1)
    q = orc.gemm("f32xf16_gguf", xn, wq, rows, qh * hd, D) + (bq if bias else 0)
    k = orc.gemm("f32xf16_gguf", xn, wk, rows, kvh * hd, D) + (bk if bias else 0)
    v = orc.gemm("f32xf16_gguf", xn, wv, rows, kvh * hd, D) + (bv if bias else 0)
    for r in range(rows):
        pos, seq = int(lens[r]), int(ids[r])
        want_q = orc.rope(q[r:r + 1].astype(np.float32), qh, hd, pos, base, 1.0, layout)[0]
        want_k = orc.rope(k[r:r + 1].astype(np.float32), kvh, hd, pos, base, 1.0, layout)[0]
        sq = np.abs(want_q).max()
        close(got_q[r] / sq, want_q / sq)
        gk, gv = kv.read_token(seq, pos)
        sk = np.abs(want_k).max()
        close(gk.view(np.float16).astype(np.float32) / sk, want_k / sk)       # f16 storage: half a step
        sv = np.abs(v[r]).max()
        close(gv.view(np.float16).astype(np.float32) / sv, v[r] / sv)
        # nothing but the row's own position was written
        if pos + 1 < S:
            ok, _ = kv.read_token(seq, pos + 1)
            assert not ok.any()
    kv.destroy()


def test_batched_greedy_step_and_lm_head(dev, orc):
    rng = np.random.default_rng(3)
    rows, V, D = 6, 5000, 256
    x = _rows_case(rng, rows, D)
    nw = (1 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    W = f16bits(rng.standard_normal((V, D)) * 0.05)
    table = f16bits(rng.standard_normal((V, D)))
    dx, dnw, dW, dT = dev.up(x), dev.up(nw), dev.up(W), dev.up(table)
    logits = dev.zeros(rows * V * 4)
    dev.call("m40llm_ext_batched_norm_gemm_f32xf16_async", dx.ptr, dnw.ptr, 1, 1e-5, dW.ptr, logits.ptr, rows, V, D)
    dev.sync()
    lg = logits.download(np.float32, (rows, V))
    want = orc.gemm("f32xf16_gguf", orc.rms_norm(x, 1e-5, nw, 1), W, rows, V, D)
    sc = np.abs(want).max(axis=1, keepdims=True)
    close(lg / sc, want / sc)
    lg[4, 100] = lg[4, 4000] = lg[4].max() + 1.0            # exact tie: the lower index wins, gap 0
    logits.upload(lg)
    cap = 3
    state = np.zeros(2 + rows, dtype=np.uint32); state[1] = cap; state[2:] = 1
    lens = np.arange(10, 10 + rows, dtype=np.uint32)
    dstate, dlens = dev.up(state), dev.up(lens)
    dids, dgaps = dev.zeros(rows * cap * 4), dev.zeros(rows * cap * 4)
    xout = dev.zeros(rows * D * 4)
    dev.call("m40llm_ext_batched_greedy_step_async", logits.ptr, rows, V, dstate.ptr, dlens.ptr, dids.ptr, dgaps.ptr, dT.ptr, D,
             xout.ptr)
    dev.sync()
    ids = dids.download(np.uint32, (rows, cap)); gaps = dgaps.download(np.float32, (rows, cap))
    xo = xout.download(np.float32, (rows, D))
    assert np.array_equal(dlens.download(np.uint32, (rows,)), lens + 1)
    assert np.array_equal(dstate.download(np.uint32, state.shape)[2:], np.full(rows, 2))
    for r in range(rows):
        tok = orc.sample_greedy(lg[r])
        assert ids[r, 1] == tok == int(np.argmax(lg[r]))
        srt = np.sort(lg[r])
        assert gaps[r, 1] == srt[-1] - srt[-2]
        assert np.array_equal(xo[r], table[tok].view(np.float16).astype(np.float32))
    assert ids[4, 1] == 100 and gaps[4, 1] == 0.0


@pytest.mark.parametrize("V", [151936, 16388, 32000])
def test_batched_greedy_step_wide_rows(dev, orc, V):
    """Rows of 16384 logits and more are reduced by several workgroups per row and merged by a second launch: the pick
    is the first index of the maximum (ties inside one part and across parts), the gap is top-1 minus top-2."""
    rng = np.random.default_rng(V)
    rows, D, cap = 5, 64, 2
    lg = rng.standard_normal((rows, V)).astype(np.float32)
    top = float(lg.max()) + 1.0
    lg[0, V - 1] = top                                       # last element of the last part
    lg[1, 7] = lg[1, V // 2 + 3] = lg[1, V - 5] = top        # tie across parts: index 7 wins, gap 0
    lg[2, 4001] = lg[2, 4002] = top                          # tie inside one part
    lg[3, :] = -np.inf; lg[3, V // 3] = -1e30                # a single finite value
    table = f16bits(rng.standard_normal((V, D)))
    logits, dT = dev.up(lg), dev.up(table)
    state = np.zeros(2 + rows, dtype=np.uint32); state[1] = cap
    lens = np.arange(3, 3 + rows, dtype=np.uint32)
    dstate, dlens = dev.up(state), dev.up(lens)
    dids, dgaps, xout = dev.zeros(rows * cap * 4), dev.zeros(rows * cap * 4), dev.zeros(rows * D * 4)
    for step in range(2):                                    # the second call reuses the scratch of the first
        dev.call("m40llm_ext_batched_greedy_step_async", logits.ptr, rows, V, dstate.ptr, dlens.ptr, dids.ptr, dgaps.ptr,
                 dT.ptr, D, xout.ptr)
    dev.sync()
    ids = dids.download(np.uint32, (rows, cap)); gaps = dgaps.download(np.float32, (rows, cap))
    xo = xout.download(np.float32, (rows, D))
    assert np.array_equal(dlens.download(np.uint32, (rows,)), lens + 2)
    assert np.array_equal(dstate.download(np.uint32, state.shape)[2:], np.full(rows, 2))
    for r in range(rows):
        tok = orc.sample_greedy(lg[r])
        assert ids[r, 0] == ids[r, 1] == tok == int(np.argmax(lg[r]))
        srt = np.sort(lg[r])
        assert gaps[r, 0] == gaps[r, 1] == srt[-1] - srt[-2]
        assert np.array_equal(xo[r], table[tok].view(np.float16).astype(np.float32))
    assert ids[1, 0] == 7 and gaps[1, 0] == 0.0 and ids[2, 0] == 4001 and ids[3, 0] == V // 3 and gaps[3, 0] == np.inf
