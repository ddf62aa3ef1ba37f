"""fp16-K / q4-V compressed cache and block-select attention: HIP path vs the CPU oracle (through the C-ABI)."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from gpu_common import close, f16bits, m40  # noqa: E402


@pytest.fixture(scope="module")
def dev():
    from gpu_common import Dev
    d = Dev()
    yield d
    d.sync()


def _read_state(kv, seq):
    B, S, H, D, W = kv.max_batch, kv.max_seq_len, kv.kv_heads, kv.head_dim, kv.compressed["recent_window"]
    return dict(
        old_k=kv.read_raw(0, np.uint16, (B, S, H, D))[seq],
        q4_v=kv.read_raw(1, np.uint8, (B, S, H, D // 2))[seq],
        q4_scale=kv.read_raw(2, np.float32, (B, S, H))[seq],
        recent_k=kv.read_raw(3, np.uint16, (B, W, H, D))[seq],
        recent_v=kv.read_raw(4, np.uint16, (B, W, H, D))[seq],
        seq_map=kv.read_raw(5, np.uint32, (B,))[seq])


def _oracle_state(c, seq):
    return dict(old_k=c.old_k[seq], q4_v=c.q4_v[seq], q4_scale=c.q4_scale[seq], recent_k=c.recent_k[seq],
                recent_v=c.recent_v[seq], seq_map=c.seq_map[seq])


@pytest.mark.parametrize("hd", [64, 128])
def test_compressed_append_evict_bit_exact(dev, orc, hd):
    rng = np.random.default_rng(hd)
    kvh, W, bs, L, S = 2, 4, 4, 11, 16
    kv = m40.KVCache(dev.ctx, S, 2, kvh, hd, dict(recent_window=W, block_size=bs, top_blocks=3))
    c = orc.CompressedKV(S, 2, kvh, hd, W, bs)
    for p in range(L):
        k = rng.standard_normal(kvh * hd).astype(np.float32); v = rng.standard_normal(kvh * hd).astype(np.float32)
        if p == 3:
            v[:hd] = 0.0                       # all-zero V row: scale 1/7
        dk, dv = dev.up(k), dev.up(v)
        # freq_scale 0 makes RoPE the identity, as the reference's own q4 tests do
        dev.call("m40llm_kvcache_append_token_f32_rope_k_at_layout_async", kv.h, 1, dk.ptr, dv.ptr, p, 0, 1e4, 0.0, 0)
        assert c.append(1, p, k, v, 1e4, 0.0, 0) == 0
    got, want = _read_state(kv, 1), _oracle_state(c, 1)
    for name in want:
        assert np.array_equal(got[name], want[name]), name
    assert not _read_state(kv, 0)["old_k"].any()
    # byte accounting literals of tests/attention_parity_cuda_grid.rs:726-843 (hd 128, max_seq 16, 1 seq, 2 heads)
    if hd == 128:
        assert (S * 1 * kvh * hd * 2, S * 1 * kvh * hd // 2, S * 1 * kvh * 4) == (8192, 2048, 128)
    # with rotation: ring rows within f16 tolerance of the oracle's rotation, V exact
    kv2 = m40.KVCache(dev.ctx, S, 1, kvh, hd, dict(recent_window=W, block_size=bs))
    c2 = orc.CompressedKV(S, 1, kvh, hd, W, bs)
    for layout in (0, 1):
        for p in range(6):
            k = rng.standard_normal(kvh * hd).astype(np.float32); v = rng.standard_normal(kvh * hd).astype(np.float32)
            dk, dv = dev.up(k), dev.up(v)
            dev.call("m40llm_kvcache_append_token_f32_rope_k_at_layout_async", kv2.h, 0, dk.ptr, dv.ptr, p, 0, 1e4, 1.0, layout)
            c2.append(0, p, k, v, 1e4, 1.0, layout)
        g, w = _read_state(kv2, 0), _oracle_state(c2, 0)
        assert np.array_equal(g["recent_v"], w["recent_v"]) and g["seq_map"] == w["seq_map"]
        close(g["recent_k"].view(np.float16).astype(np.float32), w["recent_k"].view(np.float16).astype(np.float32))
    dk, dv = dev.up(k), dev.up(v)
    dev.call("m40llm_kvcache_append_token_f32_rope_k_at_layout_async", kv.h, 2, dk.ptr, dv.ptr, 0, 0, 1e4, 1.0, 0, expect=-3)
    dev.call("m40llm_kvcache_append_token_f32_rope_k_at_layout_async", kv.h, 0, dk.ptr, dv.ptr, S, 0, 1e4, 1.0, 0, expect=-5)
    dense = m40.KVCache(dev.ctx, S, 1, kvh, hd)
    dev.call("m40llm_kvcache_append_token_f32_rope_k_compressed_at_layout_async", dense.h, 0, dk.ptr, dv.ptr, 0, 1e4, 1.0, 0, expect=-2)


@pytest.mark.parametrize("hd", [64, 128])
def test_group32_v_format_append_evict_and_bulk_fill_bit_exact(dev, orc, hd):
    """Old-store format 3 (V 4-bit in groups of 32 under an f16 scale and an f16 minimum): evictions and bulk fill write
    the oracle's bytes -- nibbles, scale | min words, K rows -- including constant groups (scale 0) and a zero row."""
    rng = np.random.default_rng(300 + hd)
    kvh, W, bs, L, S = 2, 4, 4, 13, 16
    G = hd // 32
    fmt = dict(recent_window=W, block_size=bs, top_blocks=3, exact_old_backing=3)
    kv = m40.KVCache(dev.ctx, S, 2, kvh, hd, fmt)
    c = orc.CompressedKV(S, 2, kvh, hd, W, bs, v_format=1)
    for p in range(L):
        k = rng.standard_normal(kvh * hd).astype(np.float32); v = (3.0 * rng.standard_normal(kvh * hd)).astype(np.float32)
        if p == 2:
            v[:hd] = 0.0                       # all-zero row: scale 0, every nibble 0, value = min = 0
        if p == 3:
            v[32:64] = 1.25                    # one constant group
        if p == 4:
            v[:32] = np.linspace(-2.0, 1.75, 32)   # a group on an exact grid
        dk, dv = dev.up(k), dev.up(v)
        dev.call("m40llm_kvcache_append_token_f32_rope_k_at_layout_async", kv.h, 1, dk.ptr, dv.ptr, p, 0, 1e4, 0.0, 0)
        assert c.append(1, p, k, v, 1e4, 0.0, 0) == 0

    def state(cache):
        B = cache.max_batch
        return dict(old_k=cache.read_raw(0, np.uint16, (B, S, kvh, hd)), q4_v=cache.read_raw(1, np.uint8, (B, S, kvh, hd // 2)),
                    q4_dm=cache.read_raw(2, np.uint32, (B, S, kvh, G)), recent_v=cache.read_raw(4, np.uint16, (B, W, kvh, hd)),
                    seq_map=cache.read_raw(5, np.uint32, (B,)))
    got = state(kv)
    assert np.array_equal(got["old_k"][1], c.old_k[1]) and np.array_equal(got["q4_v"][1], c.q4_v[1])
    assert np.array_equal(got["q4_dm"][1], c.q4_dm[1]) and np.array_equal(got["recent_v"][1], c.recent_v[1])
    assert got["seq_map"][1] == L and not got["q4_v"][0].any() and not got["q4_dm"][0].any()
    # bytes per (token, kv head): hd / 2 nibble bytes + 4 per group = 80 at head_dim 128 (68 in the reference's format)
    assert hd // 2 + 4 * G == (80 if hd == 128 else 40)
    # bulk fill = the same rows appended in order = the oracle's bulk fill
    L2 = 11
    k16 = f16bits(rng.standard_normal((L2, kvh, hd))); v16 = f16bits(2.0 * rng.standard_normal((L2, kvh, hd)))
    a = m40.KVCache(dev.ctx, S, 1, kvh, hd, fmt)
    dk, dv = dev.up(k16), dev.up(v16)
    dev.call("m40llm_ext_kvcache_bulk_fill_f16", a.h, 0, dk.ptr, dv.ptr, L2)
    c2 = orc.CompressedKV(S, 1, kvh, hd, W, bs, v_format=1); c2.bulk_fill(0, k16, v16)
    ga = state(a)
    assert np.array_equal(ga["old_k"][0], c2.old_k[0]) and np.array_equal(ga["q4_v"][0], c2.q4_v[0])
    assert np.array_equal(ga["q4_dm"][0], c2.q4_dm[0]) and np.array_equal(ga["recent_v"][0], c2.recent_v[0])
    dev.call("m40llm_kvcache_reset", a.h)
    assert not state(a)["q4_dm"].any()


@pytest.mark.parametrize("qh,kvh,hd,L,W,bs,top", [
    (4, 2, 128, 16, 4, 4, 3),
    (8, 2, 64, 300, 32, 16, 4),
    (6, 2, 128, 777, 100, 48, 5),
    (32, 8, 128, 4096, 512, 64, 64),
    (32, 8, 128, 32768, 512, 64, 64),      # BASELINE config 5 as written: V in groups of 32 with scale and minimum
])
def test_block_select_group32_v_format_vs_oracle(dev, orc, qh, kvh, hd, L, W, bs, top):
    r = _block_select_case(dev, orc, qh, kvh, hd, L, W, bs, top, seed=7, backing=3)
    assert np.array_equal(r["cnt"], r["wcnt"])
    assert np.array_equal(r["sel"], r["wsel"])            # the selection reads K only: same ids as the reference order
    close(r["got"], r["want"])                            # 1e-3 relative / 1e-4 absolute


def test_bulk_fill_equals_ordered_appends(dev, orc):
    rng = np.random.default_rng(2)
    kvh, hd, W, bs, S = 2, 64, 8, 4, 64
    for L in (5, 8, 9, 40):
        k16 = f16bits(rng.standard_normal((L, kvh, hd))); v16 = f16bits(rng.standard_normal((L, kvh, hd)))
        a = m40.KVCache(dev.ctx, S, 1, kvh, hd, dict(recent_window=W, block_size=bs))
        b = m40.KVCache(dev.ctx, S, 1, kvh, hd, dict(recent_window=W, block_size=bs))
        dk, dv = dev.up(k16), dev.up(v16)
        dev.call("m40llm_ext_kvcache_bulk_fill_f16", a.h, 0, dk.ptr, dv.ptr, L)
        for p in range(L):
            kf = k16[p].view(np.float16).astype(np.float32).reshape(-1); vf = v16[p].view(np.float16).astype(np.float32).reshape(-1)
            dkp, dvp = dev.up(kf), dev.up(vf)
            dev.call("m40llm_kvcache_append_token_f32_rope_k_at_layout_async", b.h, 0, dkp.ptr, dvp.ptr, p, 0, 1e4, 0.0, 0)
        ga, gb = _read_state(a, 0), _read_state(b, 0)
        for name in ga:
            assert np.array_equal(ga[name], gb[name]), (L, name)
        c = orc.CompressedKV(S, 1, kvh, hd, W, bs)
        c.bulk_fill(0, k16, v16)
        wo = _oracle_state(c, 0)
        for name in ga:
            assert np.array_equal(ga[name], wo[name]), (L, name)


def _block_select_case(dev, orc, qh, kvh, hd, L, W, bs, top, S=None, seed=0, scale_k=1.0, backing=2):
    rng = np.random.default_rng(seed)
    S = S or L
    k16 = f16bits(rng.standard_normal((L, kvh, hd)) * scale_k); v16 = f16bits(rng.standard_normal((L, kvh, hd)))
    q = rng.standard_normal((qh, hd)).astype(np.float32)
    kv = m40.KVCache(dev.ctx, S, 1, kvh, hd, dict(recent_window=W, block_size=bs, top_blocks=top, exact_old_backing=backing))
    dk, dv = dev.up(k16), dev.up(v16)
    dev.call("m40llm_ext_kvcache_bulk_fill_f16", kv.h, 0, dk.ptr, dv.ptr, L)
    c = orc.CompressedKV(S, 1, kvh, hd, W, bs, v_format=1 if backing == 3 else 0)
    c.bulk_fill(0, k16, v16)
    dq, out = dev.up(q), dev.zeros(qh * hd * 4)
    dev.call("m40llm_attention_last_token_f32_gqa_block_select_exact_fp16_k_q4_v_old_direct_async",
             kv.h, 0, dq.ptr, qh, L, W, bs, top, out.ptr)
    dev.sync()
    got = out.download(np.float32, (qh * hd,))
    sel = np.zeros((qh, 64), dtype=np.uint32); cnt = np.zeros(qh, dtype=np.uint32); ssc = np.zeros((qh, 64), dtype=np.float32)
    dev.call("m40llm_ext_block_select_read_selection", kv.h, 0, dq.ptr, qh, L, W, bs, top,
             sel.ctypes.data, cnt.ctypes.data, ssc.ctypes.data)
    orc.set_threads(8)
    # score order 0 = the reference kernel's own order (cuda/kernels.cu:2893-2912: per dimension over the block's
    # tokens, then the 128-slot halving tree), which the HIP kernel reproduces bit for bit
    rc, want, wsel, wcnt = c.attention(0, q, qh, L, top, score_order=0)
    assert rc == 0
    return dict(got=got, want=want, sel=sel, cnt=cnt, ssc=ssc, wsel=wsel, wcnt=wcnt, c=c, q=q, kv=kv, k16=k16, v16=v16)


@pytest.mark.parametrize("qh,kvh,hd,L,W,bs,top", [
    (4, 2, 128, 16, 4, 4, 3),          # tests/attention_parity_cuda_grid.rs:726-843
    (4, 2, 128, 5, 4, 32, 8),          # :608-723, one partial old block
    (8, 2, 64, 300, 32, 16, 4),
    (8, 2, 64, 20, 32, 16, 4),         # shorter than the window: no old blocks
    (32, 8, 128, 4096, 512, 64, 64),   # BASELINE config 5 geometry at 4K context
    (16, 4, 64, 2100, 1024, 32, 8),    # the reference's default window / block / top
    (6, 2, 128, 777, 100, 48, 5),      # ragged everything, partial last block
    (32, 8, 128, 32768, 512, 64, 64),  # BASELINE config 5 at its full context: 504 old blocks per kv head
])
def test_block_select_indices_exact_and_output(dev, orc, qh, kvh, hd, L, W, bs, top):
    r = _block_select_case(dev, orc, qh, kvh, hd, L, W, bs, top)
    assert np.array_equal(r["cnt"], r["wcnt"])
    assert np.array_equal(r["sel"], r["wsel"])            # block ids bit-exact vs the reference order, in rank order
    close(r["got"], r["want"])                            # 1e-3 relative / 1e-4 absolute
    # scores of the selected blocks carry the reference order's bits, and the ids are its own top-k
    c, q = r["c"], r["q"]
    tight = []
    for h in range(qh):
        s0 = c.block_scores(0, q[h], h // (qh // kvh), L, 0, W, bs)
        n = int(r["cnt"][h])
        assert np.array_equal(r["ssc"][h, :n], s0[r["sel"][h, :n]])
        b0, _ = orc.select_top_blocks(s0, top)
        assert np.array_equal(b0, r["sel"][h, :len(b0)])
        # how close the cut is in exact arithmetic: gap between the last listed and the first unlisted block
        s64 = np.sort(c.block_scores(0, q[h], h // (qh // kvh), L, 1, W, bs))[::-1]
        if len(s64) > n > 0:
            tight.append((float(s64[n - 1] - s64[n]) / max(abs(float(s64[0])), 1e-30), h))
    if tight:
        g, h = min(tight)
        print(f"[block-select L={L}] smallest float64 cut gap (relative to the top score): {g:.3e} at head {h}; "
              f"heads under 1e-6: {[hh for gg, hh in tight if gg < 1e-6]}")


@pytest.mark.parametrize("backing", [None, 3])
def test_block_select_multi_slot_batch4_32k_vs_oracle(dev, orc, backing):
    """BASELINE config 5 at batch 4: 32 q / 8 kv heads, hd 128, context 32768, 64-token blocks, top 64 + 512 recent,
    four slots with different seeds through the multi-slot entry point; outputs vs the oracle per slot, block ids exact.
    backing None: the reference's q4 V (f32 scale per token and head); 3: V in groups of 32 with f16 scale and minimum,
    the format the config names."""
    qh, kvh, hd, L, W, bs, top, nseq = 32, 8, 128, 32768, 512, 64, 64, 4
    fmt = dict(recent_window=W, block_size=bs, top_blocks=top)
    if backing is not None:
        fmt["exact_old_backing"] = backing
    kv = m40.KVCache(dev.ctx, L, nseq, kvh, hd, fmt)
    q = np.zeros((nseq, qh, hd), dtype=np.float32)
    caches = []
    for sq in range(nseq):
        rng = np.random.default_rng(100 + sq)
        k16 = f16bits(rng.standard_normal((L, kvh, hd), dtype=np.float32)); v16 = f16bits(rng.standard_normal((L, kvh, hd), dtype=np.float32))
        q[sq] = rng.standard_normal((qh, hd)).astype(np.float32)
        dk, dv = dev.up(k16), dev.up(v16)
        dev.call("m40llm_ext_kvcache_bulk_fill_f16", kv.h, sq, dk.ptr, dv.ptr, L)
        dk.free(); dv.free()
        c = orc.CompressedKV(L, 1, kvh, hd, W, bs, v_format=1 if backing == 3 else 0)
        c.bulk_fill(0, k16, v16)
        caches.append(c)
    order = np.array([2, 0, 3, 1], dtype=np.uint32)
    lens = np.full(nseq, L, dtype=np.uint32)
    dq = dev.up(np.ascontiguousarray(q[order]))
    out = dev.zeros(q.nbytes)
    dev.call("m40llm_ext_attention_block_select_fp16_k_q4_v_multi_async", kv.h, nseq, order.ctypes.data_as(C.c_void_p),
             lens.ctypes.data_as(C.c_void_p), dq.ptr, qh, W, bs, top, out.ptr)
    dev.sync()
    got = out.download(np.float32, (nseq, qh * hd))
    orc.set_threads(16)
    for i, sq in enumerate(order):
        rc, want, wsel, wcnt = caches[sq].attention(0, q[sq], qh, L, top, score_order=0)
        assert rc == 0
        close(got[i], want)
        sel = np.zeros((qh, 64), dtype=np.uint32); cnt = np.zeros(qh, dtype=np.uint32)
        dev.call("m40llm_ext_block_select_read_selection", kv.h, int(sq), dq.ptr + i * qh * hd * 4, qh, L, W, bs, top,
                 sel.ctypes.data, cnt.ctypes.data, None)
        assert np.array_equal(cnt, wcnt) and np.array_equal(sel, wsel), int(sq)
    kv.destroy()


def test_block_select_all_blocks_equals_dense(dev, orc):
    # property of tests/attention_parity_cuda_grid.rs:182-486: top >= old_blocks -> every token attended
    qh, kvh, hd, L, W, bs = 8, 2, 64, 200, 40, 8
    r = _block_select_case(dev, orc, qh, kvh, hd, L, W, bs, 64, seed=3)
    assert list(r["cnt"]) == [20] * qh
    k = r["k16"].view(np.float16).astype(np.float64); q = r["q"].astype(np.float64)
    # dequantised V via the oracle cache
    c = r["c"]
    vq = np.zeros((L, kvh, hd))
    for t in range(L):
        for h in range(kvh):
            if t < L - W:
                p = c.q4_v[0, t, h]; s = c.q4_scale[0, t, h]
                nib = np.stack([p & 15, p >> 4], axis=1).reshape(-1).astype(np.int32)
                nib = np.where(nib >= 8, nib - 16, nib)
                vq[t, h] = (nib.astype(np.float32) * s).astype(np.float16).astype(np.float64)
            else:
                vq[t, h] = r["v16"][t, h].view(np.float16).astype(np.float64)
    for h in range(qh):
        kvhh = h // (qh // kvh)
        s = (k[:, kvhh] @ q[h]) * 0.125
        p = np.exp(s - s.max()); p /= p.sum()
        close(r["got"][h * hd:(h + 1) * hd], p @ vq[:, kvhh])


def test_block_select_ties_and_degenerate_scores(dev, orc):
    # identical K rows everywhere -> every block scores the same -> lowest block ids win, in ascending order
    qh, kvh, hd, L, W, bs, top = 4, 2, 64, 8 + 16 * 6, 8, 16, 3
    rng = np.random.default_rng(4)
    row = rng.standard_normal((1, kvh, hd))
    k16 = f16bits(np.repeat(row, L, axis=0)); v16 = f16bits(rng.standard_normal((L, kvh, hd)))
    q = rng.standard_normal((qh, hd)).astype(np.float32)
    kv = m40.KVCache(dev.ctx, L, 1, kvh, hd, dict(recent_window=W, block_size=bs))
    dk, dv = dev.up(k16), dev.up(v16)
    dev.call("m40llm_ext_kvcache_bulk_fill_f16", kv.h, 0, dk.ptr, dv.ptr, L)
    dq = dev.up(q)
    sel = np.zeros((qh, 64), dtype=np.uint32); cnt = np.zeros(qh, dtype=np.uint32)
    dev.call("m40llm_ext_block_select_read_selection", kv.h, 0, dq.ptr, qh, L, W, bs, top, sel.ctypes.data, cnt.ctypes.data, None)
    assert list(cnt) == [3] * qh and all(list(sel[h, :3]) == [0, 1, 2] for h in range(qh))
    c = orc.CompressedKV(L, 1, kvh, hd, W, bs); c.bulk_fill(0, k16, v16)
    _, _, wsel, _ = c.attention(0, q, qh, L, top, score_order=0)
    assert np.array_equal(sel, wsel)


def test_block_select_argument_checks(dev, orc):
    qh, kvh, hd, L, W, bs = 4, 2, 64, 64, 16, 8
    kv = m40.KVCache(dev.ctx, L, 1, kvh, hd, dict(recent_window=W, block_size=bs))
    dense = m40.KVCache(dev.ctx, L, 1, kvh, hd)
    q = dev.up(np.zeros(qh * hd, dtype=np.float32)); out = dev.zeros(qh * hd * 4)
    f = "m40llm_attention_last_token_f32_gqa_block_select_exact_fp16_k_q4_v_old_direct_async"
    dev.call(f, kv.h, 0, None, qh, L, W, bs, 4, out.ptr, expect=-1)
    dev.call(f, dense.h, 0, q.ptr, qh, L, W, bs, 4, out.ptr, expect=-16)      # missing backing
    dev.call(f, kv.h, 1, q.ptr, qh, L, W, bs, 4, out.ptr, expect=-2)
    dev.call(f, kv.h, 0, q.ptr, qh, 0, W, bs, 4, out.ptr, expect=-3)
    dev.call(f, kv.h, 0, q.ptr, qh, L + 1, W, bs, 4, out.ptr, expect=-3)
    dev.call(f, kv.h, 0, q.ptr, 3, L, W, bs, 4, out.ptr, expect=-4)
    dev.call(f, kv.h, 0, q.ptr, qh, L, 0, bs, 4, out.ptr, expect=-6)
    dev.call(f, kv.h, 0, q.ptr, qh, L, W, 0, 4, out.ptr, expect=-6)
    dev.call(f, kv.h, 0, q.ptr, qh, L, W, bs, 0, out.ptr, expect=-6)
    dev.call(f, kv.h, 0, q.ptr, qh, L, W, bs, 65, out.ptr, expect=-6)          # top_blocks > 64
    assert dev.lib.m40llm_kvcache_create_compressed(dev.h, 16, 1, 2, 64, 0, 4, 1, 0, 0, 2) is None
    assert dev.lib.m40llm_kvcache_create_compressed(dev.h, 16, 1, 2, 80, 4, 4, 1, 0, 0, 2) is None


@pytest.mark.parametrize("hd", [64, 128])
def test_dense_backed_block_select(dev, orc, hd):
    rng = np.random.default_rng(5 + hd)
    qh, kvh, L, W, bs, top, S = 8, 2, 500, 64, 16, 6, 512
    k16 = f16bits(rng.standard_normal((L, kvh, hd))); v16 = f16bits(rng.standard_normal((L, kvh, hd)))
    q = rng.standard_normal((qh, hd)).astype(np.float32)
    kv = m40.KVCache(dev.ctx, S, 1, kvh, hd)
    dev.fill_dense(kv, 0, k16, v16)
    dq, out = dev.up(q), dev.zeros(qh * hd * 4)
    dev.call("m40llm_attention_last_token_f32_gqa_block_select_exact_async", kv.h, 0, dq.ptr, qh, L, W, bs, top, out.ptr)
    dev.sync()
    Kc = np.zeros((1, S, kvh, hd), dtype=np.uint16); Vc = np.zeros_like(Kc)
    Kc[0, :L] = k16; Vc[0, :L] = v16
    rc, want, wsel, wcnt = orc.dense_block_select(Kc, Vc, S, kvh, hd, 0, q, qh, L, W, bs, top, 0)
    assert rc == 0
    close(out.download(np.float32, (qh * hd,)), want)
    sel = np.zeros((qh, 64), dtype=np.uint32); cnt = np.zeros(qh, dtype=np.uint32)
    dev.call("m40llm_ext_block_select_read_selection", kv.h, 0, dq.ptr, qh, L, W, bs, top, sel.ctypes.data, cnt.ctypes.data, None)
    assert np.array_equal(sel, wsel) and np.array_equal(cnt, wcnt)
    # every block selected -> dense attention
    dev.call("m40llm_attention_last_token_f32_gqa_block_select_exact_async", kv.h, 0, dq.ptr, qh, L, W, bs, 64, out.ptr)
    dev.sync()
    close(out.download(np.float32, (qh * hd,)), dev.attention(kv, 0, q, qh, L))


def test_debug_select_old_blocks_host_twin(dev, orc):
    rng = np.random.default_rng(6)
    kvh, hd, W, bs, L = 2, 64, 8, 4, 8 + 4 * 9 + 2
    k16 = f16bits(rng.standard_normal((L, kvh, hd)))
    kv = m40.KVCache(dev.ctx, 64, 1, kvh, hd, dict(recent_window=W, block_size=bs))
    dk = dev.up(k16)
    dev.call("m40llm_ext_kvcache_bulk_fill_f16", kv.h, 0, dk.ptr, dk.ptr, L)
    c = orc.CompressedKV(64, 1, kvh, hd, W, bs); c.bulk_fill(0, k16, k16)
    q = rng.standard_normal(4 * hd).astype(np.float32); dq = dev.up(q)
    blocks = np.zeros(2048, dtype=np.uint32); scores = np.zeros(2048, dtype=np.float32)
    start = np.zeros(2048, dtype=np.uint32); end = np.zeros(2048, dtype=np.uint32)
    count = np.zeros(1, dtype=np.uint32); total = np.zeros(1, dtype=np.uint32)
    dev.call("m40llm_kvcache_debug_select_old_blocks", kv.h, 0, dq.ptr, 4, L, 999, 999, 3,
             blocks.ctypes.data, scores.ctypes.data, start.ctypes.data, end.ctypes.data, count.ctypes.data, 2048, total.ctypes.data)
    rc, wb, ws, wst, wen, wtot = c.debug_select(0, q[:hd], L, 3)
    n = int(count[0])
    assert rc == 0 and n == len(wb) == 3 and total[0] == wtot == 10
    assert np.array_equal(blocks[:n], wb) and np.array_equal(scores[:n], ws)
    assert np.array_equal(start[:n], wst) and np.array_equal(end[:n], wen)


def test_multi_slot_call_equals_per_slot_calls(dev, orc):
    """Several sequences in one set of launches: same bits as one call per sequence (different lengths, one sequence
    still without old blocks)."""
    rng = np.random.default_rng(21)
    qh, kvh, hd, W, bs, top, S = 8, 2, 128, 16, 8, 5, 200
    nseq = 4
    lens = np.array([200, 9, 77, 130], dtype=np.uint32)
    kv = m40.KVCache(dev.ctx, S, nseq, kvh, hd, compressed=dict(recent_window=W, block_size=bs, top_blocks=top))
    for s in range(nseq):
        k16 = f16bits(rng.standard_normal((int(lens[s]), kvh, hd))); v16 = f16bits(rng.standard_normal((int(lens[s]), kvh, hd)))
        dk, dv = dev.up(k16), dev.up(v16)
        dev.call("m40llm_ext_kvcache_bulk_fill_f16", kv.h, s, dk.ptr, dv.ptr, int(lens[s]))
    q = rng.standard_normal((nseq, qh * hd)).astype(np.float32)
    dq = dev.up(q)
    single = dev.zeros(q.nbytes); multi = dev.zeros(q.nbytes)
    name = "m40llm_attention_last_token_f32_gqa_block_select_exact_fp16_k_q4_v_old_direct_async"
    order = np.array([2, 0, 3, 1], dtype=np.uint32)          # slots in arbitrary order
    for i, s in enumerate(order):
        dev.call(name, kv.h, int(s), dq.ptr + i * qh * hd * 4, qh, int(lens[s]), W, bs, top, single.ptr + i * qh * hd * 4)
    ids = order.copy(); ls = lens[order].copy()
    dev.call("m40llm_ext_attention_block_select_fp16_k_q4_v_multi_async", kv.h, nseq, ids.ctypes.data_as(C.c_void_p),
             ls.ctypes.data_as(C.c_void_p), dq.ptr, qh, W, bs, top, multi.ptr)
    dev.sync()
    a = single.download(np.float32, q.shape); b = multi.download(np.float32, q.shape)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert np.isfinite(a).all() and np.abs(a).max() > 0
    # the same slot twice, too many slots
    ids2 = np.array([1, 1], dtype=np.uint32)
    dev.call("m40llm_ext_attention_block_select_fp16_k_q4_v_multi_async", kv.h, 2, ids2.ctypes.data_as(C.c_void_p),
             ls.ctypes.data_as(C.c_void_p), dq.ptr, qh, W, bs, top, multi.ptr, expect=-2)
    dev.call("m40llm_ext_attention_block_select_fp16_k_q4_v_multi_async", kv.h, 9, ids.ctypes.data_as(C.c_void_p),
             ls.ctypes.data_as(C.c_void_p), dq.ptr, qh, W, bs, top, multi.ptr, expect=-2)
    kv.destroy()
