"""Packed prefill through the host layer: the one-launch RoPE + bias + KV append against the reference's per-token
call sequence (bit-exact), and the whole prefill forward against the CPU oracle stepping token by token."""
import ctypes as C
import importlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from gpu_common import Dev, close, m40  # noqa: E402

syn = importlib.import_module("m40-llm_amd.synthetic")


@pytest.fixture(scope="module")
def dev():
    return Dev()


def u32(a):
    return np.ascontiguousarray(a, dtype=np.uint32)


@pytest.mark.parametrize("layout,bias,hd,q_heads,kv_heads", [(0, False, 64, 4, 2), (1, True, 128, 4, 1), (1, False, 16, 2, 2)])
def test_prefill_rope_append_equals_per_token_calls(dev, layout, bias, hd, q_heads, kv_heads):
    # src/infer/forward.rs:149-160 (bias rows) + :2349-2396 (append with rotated K, RoPE on the Q row, RoPE on the K row)
    rng = np.random.default_rng(10 + hd)
    lens, slots, starts = [5, 1, 9], [2, 0, 3], [0, 7, 3]
    rows, D, KV, base = sum(lens), q_heads * hd, kv_heads * hd, 1e6 if layout else 1e4
    q = rng.standard_normal((rows, D)).astype(np.float32)
    k = rng.standard_normal((rows, KV)).astype(np.float32)
    v = rng.standard_normal((rows, KV)).astype(np.float32)
    bq, bk, bv = (rng.standard_normal(n).astype(np.float32) for n in (D, KV, KV))
    dbq, dbk, dbv = dev.up(bq), dev.up(bk), dev.up(bv)
    # one launch
    kv_a = m40.KVCache(dev.ctx, 32, 4, kv_heads, hd)
    dq, dk, dv = dev.up(q), dev.up(k), dev.up(v)
    h_slots, h_lens, h_starts = u32(slots), u32(lens), u32(starts)      # host tables must outlive the call
    dev.call("m40llm_ext_prefill_rope_append_async", kv_a.h, dq.ptr, dk.ptr, dv.ptr, 3, h_slots.ctypes.data, h_lens.ctypes.data,
             h_starts.ctypes.data, q_heads, base, 1.0, layout, dbq.ptr if bias else None, dbk.ptr if bias else None,
             dbv.ptr if bias else None)
    dev.sync()
    q_a, k_a, v_a = dq.download(np.float32, q.shape), dk.download(np.float32, k.shape), dv.download(np.float32, v.shape)
    # the per-token sequence
    kv_b = m40.KVCache(dev.ctx, 32, 4, kv_heads, hd)
    dq2, dk2, dv2 = dev.up(q), dev.up(k), dev.up(v)
    row = 0
    for s, n in enumerate(lens):
        for j in range(n):
            qr, kr, vr = dq2.ptr + row * D * 4, dk2.ptr + row * KV * 4, dv2.ptr + row * KV * 4
            if bias:
                dev.call("m40llm_residual_add_f32_async", qr, dbq.ptr, qr, D)
                dev.call("m40llm_residual_add_f32_async", kr, dbk.ptr, kr, KV)
                dev.call("m40llm_residual_add_f32_async", vr, dbv.ptr, vr, KV)
            pos = starts[s] + j
            dev.call("m40llm_kvcache_append_token_f32_rope_k_at_layout_async", kv_b.h, slots[s], kr, vr, pos, pos, base, 1.0, layout)
            dev.call("m40llm_rope_f32_inplace_layout_async", qr, 1, q_heads, hd, pos, base, 1.0, layout)
            dev.call("m40llm_rope_f32_inplace_layout_async", kr, 1, kv_heads, hd, pos, base, 1.0, layout)
            row += 1
    dev.sync()
    assert np.array_equal(q_a.view(np.uint32), dq2.download(np.float32, q.shape).view(np.uint32))
    assert np.array_equal(k_a.view(np.uint32), dk2.download(np.float32, k.shape).view(np.uint32))
    assert np.array_equal(v_a.view(np.uint32), dv2.download(np.float32, v.shape).view(np.uint32))
    for s, n in enumerate(lens):
        for j in range(n):
            ka, va = kv_a.read_token(slots[s], starts[s] + j)
            kb, vb = kv_b.read_token(slots[s], starts[s] + j)
            assert np.array_equal(ka, kb) and np.array_equal(va, vb)
    assert np.array_equal(kv_a.read_raw(5, np.uint32, (4,)), kv_b.read_raw(5, np.uint32, (4,)))
    assert kv_a.read_raw(5, np.uint32, (4,)).tolist() == [8, 0, 5, 12]
    # rotation is norm-preserving per pair and the identity at position 0 (row 0 of sequence 0 starts at 0)
    want0 = q[0] + (bq if bias else 0)
    assert np.array_equal(q_a[0], want0.astype(np.float32))
    close(np.linalg.norm(q_a, axis=1), np.linalg.norm(q + (bq if bias else 0), axis=1), 1e-5, 1e-5)


def test_prefill_rope_append_argument_checks(dev):
    kv = m40.KVCache(dev.ctx, 8, 2, 2, 64)
    z = dev.zeros(16 * 4 * 64 * 4)
    keep_one = u32([1])
    one = keep_one.ctypes.data

    def case(slots, lens, starts, expect=0):
        a, b, c = u32(slots), u32(lens), u32(starts)                    # alive until the call returns
        dev.call("m40llm_ext_prefill_rope_append_async", kv.h, z.ptr, z.ptr, z.ptr, len(slots), a.ctypes.data, b.ctypes.data,
                 c.ctypes.data, 4, 1e4, 1.0, 0, None, None, None, expect=expect)

    case([0], [8], [0])
    case([0], [8], [1], expect=-5)            # runs past max_seq_len
    case([2], [1], [0], expect=-2)            # slot out of range
    case([0, 0], [1, 1], [0, 1], expect=-8)   # one slot twice
    case([0], [0], [0], expect=-7)            # empty sequence
    dev.call("m40llm_ext_prefill_rope_append_async", kv.h, z.ptr, z.ptr, z.ptr, 0, one, one, one, 4, 1e4, 1.0, 0, None, None, None, expect=-2)
    dev.call("m40llm_ext_prefill_rope_append_async", kv.h, z.ptr, z.ptr, z.ptr, 1, one, one, one, 4, 1e4, 1.0, 0, z.ptr, None, None, expect=-2)
    dev.call("m40llm_ext_prefill_rope_append_async", kv.h, None, z.ptr, z.ptr, 1, one, one, one, 4, 1e4, 1.0, 0, None, None, None, expect=-1)
    ckv = m40.KVCache(dev.ctx, 64, 1, 2, 64, compressed=dict(recent_window=16, block_size=16))
    zero = u32([0])
    dev.call("m40llm_ext_prefill_rope_append_async", ckv.h, z.ptr, z.ptr, z.ptr, 1, zero.ctypes.data, one, None, 4, 1e4, 1.0, 0, None, None, None,
             expect=-9)
    dev.sync()


def test_embed_rows(dev):
    rng = np.random.default_rng(2)
    table = rng.standard_normal((50, 96)).astype(np.float16)
    toks = u32([3, 49, 0, 3, 17])
    dt, dtab, out = dev.up(toks), dev.up(table.view(np.uint16)), dev.zeros(5 * 96 * 4)
    dev.call("m40llm_ext_embed_rows_async", dtab.ptr, dt.ptr, 5, 50, 96, out.ptr)
    dev.sync()
    assert np.array_equal(out.download(np.float32, (5, 96)), table[toks].astype(np.float32))
    dev.call("m40llm_ext_embed_rows_async", dtab.ptr, dt.ptr, 0, 50, 96, out.ptr, expect=-2)


def _oracle_model(orc, cfg, W, max_seq, max_sequences):
    m = orc.Model(dict(cfg, qkv_bias=bool(cfg.get("qkv_bias"))), W)
    m.alloc_kv(max_seq, max_sequences)
    return m


@pytest.mark.parametrize("layout,bias,hd", [(0, False, 64), (1, True, 128)])
def test_forward_prefill_matches_token_by_token_oracle_and_decode_continues(dev, orc, layout, bias, hd):
    cfg = dict(n_layers=3, d_model=4 * hd, q_heads=4, kv_heads=2, head_dim=hd, ffn=6 * 64, vocab=500, rms_eps=1e-5,
               rope_base=1e6 if layout else 10000.0, rope_scale=1.0, rope_layout=layout, qkv_bias=bias)
    W = syn.make_weights(cfg, seed=6, std=0.08, emb_std=1.0)
    for l in range(cfg["n_layers"]):
        W["ffn_norm"][l] = (1 + 0.1 * np.random.default_rng(l).standard_normal(cfg["d_model"])).astype(np.float32)
    S = 96
    dm = syn.DeviceModel(dev.ctx, cfg, W, max_seq_len=S, max_sequences=4)
    om = _oracle_model(orc, cfg, W, S, 4)
    rng = np.random.default_rng(8)
    prompts = [rng.integers(0, 500, size=n).tolist() for n in (37, 1, 70)]      # 70 > one query tile of the attention kernel
    seqs = [2, 0, 3]
    hid, log = dm.forward_prefill(seqs, prompts)
    for i, (s, p) in enumerate(zip(seqs, prompts)):
        for pos, t in enumerate(p):
            want_h = om.token_forward(s, pos, t)
        # whole-model tolerance of the reference's own parity test (tests/forward_parity_toy.rs:389), scaled to the row
        close(hid[i], want_h, 5e-3, 5e-3 * max(1.0, np.abs(want_h).max()))
        wl = om.logits(want_h)
        assert int(np.argmax(log[i])) == int(np.argmax(wl)), i
        # the cache the prefill wrote serves the decode that follows: ids equal the oracle's continuing decode
        first = int(np.argmax(wl))
        got, gap = dm.decode_greedy(s, [first], 6, start_pos=len(p))
        want, _ = om.decode_greedy(s, [first], 6, start_pos=len(p))
        assert np.array_equal(got, want), (i, gap.min())
    # the same prompts one by one through the per-token path of the device: same next token
    for i, (s, p) in enumerate(zip(seqs, prompts)):
        for pos, t in enumerate(p):
            _, l1 = dm.forward_token(1, pos, t, want_hidden=False)
        assert int(np.argmax(l1)) == int(np.argmax(log[i]))
    with pytest.raises(RuntimeError, match="empty prompt"):
        dm.forward_prefill([0], [[]])
    with pytest.raises(RuntimeError, match="longer than max_seq_len"):
        dm.forward_prefill([0], [[1] * (S + 1)])
    dm.close()


def _f16(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32).astype(np.float16).view(np.uint16))


@pytest.mark.parametrize("kind,M,K,Ns,residual,norm_dtype", [
    (1, 300, 2048, (2048, 256, 256), False, 0),     # RMSNorm -> Q/K/V, 128 x 128 tiles, f16 norm weights
    (1, 4100, 2048, (2048, 256, 256), False, 1),    # the same on the wide tile, f32 norm weights
    (1, 40, 96, (136,), False, 0),                  # one matrix, three K steps
    (0, 300, 2048, (2048,), True, 0),               # O projection + residual: K split, residual added with the partial sums
    (0, 2100, 2048, (2048,), True, 0),              # no K split, 128 x 128 tiles: residual in the kernel's last step
    (0, 4100, 2048, (2056,), True, 0),              # wide tile, ragged N
    (2, 300, 5632, (2048,), True, 0),               # SwiGLU -> down projection + residual (a workgroup per row), K split
    (2, 4100, 5632, (2048,), True, 0),              # the same on the wide tile
    (2, 200, 256, (384, 64), False, 0),             # SwiGLU source, a wave per row, two matrices
])
def test_prefill_gemm_fused_equals_separate_calls(dev, kind, M, K, Ns, residual, norm_dtype):
    # src/infer/forward.rs:2300-2345, 2440-2530 issue rms_norm / swiglu, the GEMMs and residual_add as separate launches; the
    # fused call has to give the bits of rms_norm / swiglu -> the GEMM call over the same matrices -> residual_add, also with
    # the result written over the residual
    rng = np.random.default_rng(kind * 1000 + M + K)
    x = rng.standard_normal((M, K)).astype(np.float32)
    x[3] *= 1e-4
    x[5, ::3] *= 300.0
    x2 = rng.standard_normal((M, K)).astype(np.float32)
    wn = (1.0 + 0.1 * rng.standard_normal(K)).astype(np.float32)
    d_wn = dev.up(_f16(wn) if norm_dtype == 0 else wn)
    Bs = [_f16(rng.standard_normal((n, K)) * 0.05) for n in Ns]
    R = rng.standard_normal((M, Ns[0])).astype(np.float32)
    dx, dx2, dB, dR = dev.up(x), dev.up(x2), [dev.up(b) for b in Bs], dev.up(R)
    eps = 1e-5
    # separate calls
    rows = dev.zeros(M * K * 4)
    if kind == 1:
        dev.call("m40llm_rms_norm_f32_weighted_async", dx.ptr, d_wn.ptr, rows.ptr, M, K, eps, norm_dtype)
    elif kind == 2:
        dev.call("m40llm_swiglu_f32_async", dx.ptr, dx2.ptr, rows.ptr, M * K)
    dev.sync()
    src = rows if kind else dx
    sep = [dev.zeros(M * n * 4) for n in Ns]
    margs = []
    for i in range(3):
        margs += [dB[i].ptr, Ns[i], sep[i].ptr] if i < len(Ns) else [None, 0, None]
    dev.call("m40llm_ext_gemm_f32xf16_gguf_f32_multi_async", src.ptr, M, K, len(Ns), *margs, 0)
    dev.sync()
    if residual:
        dev.call("m40llm_residual_add_f32_async", dR.ptr, sep[0].ptr, sep[0].ptr, M * Ns[0])
        dev.sync()
    want = [sep[i].download(np.float32, (M, n)) for i, n in enumerate(Ns)]
    # one fused call
    outs = [dev.zeros(M * n * 4) for n in Ns]
    args = []
    for i in range(3):
        if i == 0:
            args += [dB[0].ptr, Ns[0], outs[0].ptr, dR.ptr if residual else None]
        elif i < len(Ns):
            args += [dB[i].ptr, Ns[i], outs[i].ptr]
        else:
            args += [None, 0, None]
    dev.call("m40llm_ext_prefill_gemm_fused_async", kind, dx.ptr, dx2.ptr if kind == 2 else None, d_wn.ptr if kind == 1 else None,
             norm_dtype, eps, M, K, len(Ns), *args, 0)
    dev.sync()
    for i, n in enumerate(Ns):
        assert np.array_equal(outs[i].download(np.float32, (M, n)).view(np.uint32), want[i].view(np.uint32)), i
    if residual:
        # result over the residual
        args[2] = dR.ptr
        dev.call("m40llm_ext_prefill_gemm_fused_async", kind, dx.ptr, dx2.ptr if kind == 2 else None, d_wn.ptr if kind == 1 else None,
                 norm_dtype, eps, M, K, len(Ns), *args, 0)
        dev.sync()
        assert np.array_equal(dR.download(np.float32, (M, Ns[0])).view(np.uint32), want[0].view(np.uint32))


def test_prefill_gemm_fused_declines_and_checks(dev):
    rng = np.random.default_rng(3)
    M, K, N = 8, 256, 64
    dx, dB, out = dev.up(rng.standard_normal((M, K)).astype(np.float32)), dev.up(_f16(rng.standard_normal((N, K)))), dev.zeros(M * N * 4)
    tail = [None, 0, None, None, 0, None]
    # few rows: not the many-row kernel's case -- nothing enqueued, the caller issues the separate calls
    dev.call("m40llm_ext_prefill_gemm_fused_async", 0, dx.ptr, None, None, 0, 1e-5, M, K, 1, dB.ptr, N, out.ptr, None, *tail, 0, expect=1)
    assert not out.download(np.float32, (M, N)).any()
    dev.call("m40llm_ext_prefill_gemm_fused_async", 3, dx.ptr, None, None, 0, 1e-5, 64, K, 1, dB.ptr, N, out.ptr, None, *tail, 0, expect=-2)
    dev.call("m40llm_ext_prefill_gemm_fused_async", 1, dx.ptr, None, None, 0, 1e-5, 64, K, 1, dB.ptr, N, out.ptr, None, *tail, 0, expect=-1)
    dev.call("m40llm_ext_prefill_gemm_fused_async", 2, dx.ptr, None, None, 0, 1e-5, 64, K, 1, dB.ptr, N, out.ptr, None, *tail, 0, expect=-1)
    dev.call("m40llm_ext_prefill_gemm_fused_async", 0, dx.ptr, None, None, 0, 1e-5, 64, K, 2, dB.ptr, N, out.ptr, out.ptr, dB.ptr, N, out.ptr,
             None, 0, None, 0, expect=-2)     # a residual needs a single matrix
