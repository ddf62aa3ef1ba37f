"""Pins the CPU oracle against evidence that does not come from the oracle itself:
literals and closed-form fixtures held by the reference's own tests, independent
implementations (numpy float16, float64 linear algebra), and invariants."""
import numpy as np
import pytest


# ---------------------------------------------------------------- f16 conversion
def test_f16_to_f32_all_codes_match_numpy(orc):
    codes = np.arange(65536, dtype=np.uint16)
    got = orc.f16_bits_to_f32(codes)
    want = codes.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f32_to_f16_rne_matches_numpy(orc):
    rng = np.random.default_rng(1)
    xs = [rng.standard_normal(200000).astype(np.float32) * s for s in (1e-8, 1e-5, 1e-3, 1.0, 300.0, 7e4)]
    # every half value, every midpoint between neighbours, and one ulp either side of them
    h = np.arange(0x7C00, dtype=np.uint16).view(np.float16).astype(np.float32)
    mids = ((h[:-1].astype(np.float64) + h[1:].astype(np.float64)) / 2).astype(np.float32)
    xs += [h, mids, np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf)),
           np.array([0.0, -0.0, np.inf, -np.inf, 65504.0, 65519.99, 65520.0, 1e38, 2.0 ** -25,
                     np.nextafter(np.float32(2.0 ** -25), np.float32(1))], dtype=np.float32)]
    x = np.concatenate(xs)
    x = np.concatenate([x, -x])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = orc.f32_to_f16_bits(x)
    assert np.array_equal(got, want)


def test_kv_append_fixtures_bit_exact(orc):
    # fixtures of tests/kv_f32_to_f16_append.rs:42-45,84-89 (odd element count 3 included)
    for elems in (3, 16):
        i = np.arange(elems, dtype=np.float32)
        for k, v in ((i + 0.25, 100 + i + 0.5), (-10 + 0.125 * i, np.float32(np.pi) + 0.25 * i)):
            k = k.astype(np.float32); v = v.astype(np.float32)
            K = np.zeros((1, 2, 1, elems), dtype=np.uint16); V = np.zeros_like(K)
            orc.lib().orc_kv_append_f32(orc.ptr(K), orc.ptr(V), 2, 1, elems, 0, 1, orc.ptr(k), orc.ptr(v))
            assert np.array_equal(K[0, 1, 0], k.astype(np.float16).view(np.uint16))
            assert np.array_equal(V[0, 1, 0], v.astype(np.float16).view(np.uint16))
            assert not K[0, 0].any()


# ---------------------------------------------------------------- layout
def test_kv_layout_reference_literals(orc):
    L = orc.lib()
    # tests/kv_layout.rs: max_seq 4, batch 2, heads 3, head_dim 5
    assert L.orc_kv_elems_per_token(3, 5) == 15
    assert L.orc_kv_base(4, 3, 5, 1, 0) == 60
    assert L.orc_kv_index(4, 3, 5, 1, 2, 2, 4) == 104


# ---------------------------------------------------------------- attention
def _f64_attention(Kf, Vf, q, q_heads, kv_heads, hd, L, inv_sqrt):
    out = np.zeros((q_heads, hd))
    g = q_heads // kv_heads
    for h in range(q_heads):
        k = Kf[:L, h // g].astype(np.float64)
        v = Vf[:L, h // g].astype(np.float64)
        s = (k @ q[h].astype(np.float64)) * inv_sqrt
        p = np.exp(s - s.max()); p /= p.sum()
        out[h] = p @ v
    return out


def _mk_cache(orc, k_f32, v_f32):
    """k_f32: [L, kvh, hd] -> f16 bits via numpy (independent RNE)"""
    return (np.ascontiguousarray(k_f32.astype(np.float16).view(np.uint16)[None]),
            np.ascontiguousarray(v_f32.astype(np.float16).view(np.uint16)[None]))


def test_attention_mha_grid_fixture_vs_float64(orc):
    # grid and closed-form data of tests/attention_parity_cpu_grid.rs:74-118
    for heads in (1, 2, 3, 4):
        for hd in (1, 5, 7, 8, 16, 31, 32, 63, 64):
            dim = heads * hd
            for L in (1, 2, 3, 4, 7, 8, 16):
                t = np.arange(L)[:, None]; i = np.arange(dim)[None, :]
                k = ((t * dim + i).astype(np.float32) * np.float32(0.01) - 1).astype(np.float32)
                v = ((t * dim + (dim - 1 - i)).astype(np.float32) * np.float32(0.02) - 2).astype(np.float32)
                q = (np.arange(dim, dtype=np.float32) * np.float32(0.003) - np.float32(0.5)).astype(np.float32)
                K, V = _mk_cache(orc, k.reshape(L, heads, hd), v.reshape(L, heads, hd))
                got = orc.attention(K, V, L, heads, hd, 0, q, heads, L).reshape(heads, hd)
                Kf = K[0].view(np.float16).astype(np.float32); Vf = V[0].view(np.float16).astype(np.float32)
                want = _f64_attention(Kf, Vf, q.reshape(heads, hd), heads, heads, hd, L,
                                      float(orc.lib().orc_inv_sqrt_head_dim(hd)))
                assert np.allclose(got, want, rtol=1e-4, atol=1e-5), (heads, hd, L)


def test_attention_gqa_config1_fixture_vs_float64(orc):
    # tests/attention_parity_cuda_grid.rs:1737-1772: 32 q heads / 4 kv heads / hd 64, L in {128, 512}
    qh, kvh, hd = 32, 4, 64
    kv_dim = kvh * hd
    for L in (128, 512):
        t = np.arange(L)[:, None]; i = np.arange(kv_dim)[None, :]
        k = ((t * kv_dim + i).astype(np.float32) * np.float32(0.0003) - np.float32(0.25))
        v = ((t * kv_dim + (kv_dim - 1 - i)).astype(np.float32) * np.float32(0.0002) - np.float32(0.1))
        q = (np.arange(qh * hd, dtype=np.float32) * np.float32(0.0004) - np.float32(0.2))
        K, V = _mk_cache(orc, k.reshape(L, kvh, hd), v.reshape(L, kvh, hd))
        got = orc.attention(K, V, L, kvh, hd, 0, q, qh, L).reshape(qh, hd)
        Kf = K[0].view(np.float16).astype(np.float32); Vf = V[0].view(np.float16).astype(np.float32)
        want = _f64_attention(Kf, Vf, q.reshape(qh, hd), qh, kvh, hd, L, 0.125)
        assert np.allclose(got, want, rtol=1e-4, atol=1e-5)


def test_attention_invariants(orc):
    rng = np.random.default_rng(3)
    qh, kvh, hd, L = 8, 2, 128, 9
    k = rng.standard_normal((L, kvh, hd)).astype(np.float32)
    v = rng.standard_normal((L, kvh, hd)).astype(np.float32)
    q = rng.standard_normal((qh, hd)).astype(np.float32)
    K, V = _mk_cache(orc, k, v)
    Vf = V[0].view(np.float16).astype(np.float32)
    # L = 1 -> output is the V row of the mapped kv head, exactly
    got = orc.attention(K, V, L, kvh, hd, 0, q, qh, 1).reshape(qh, hd)
    for h in range(qh):
        assert np.array_equal(got[h], Vf[0, h // (qh // kvh)])
    # identical K rows -> uniform weights -> mean of V
    k2 = np.repeat(k[:1], L, axis=0)
    K2, _ = _mk_cache(orc, k2, v)
    got = orc.attention(K2, V, L, kvh, hd, 0, q, qh, L).reshape(qh, hd)
    for h in range(qh):
        assert np.allclose(got[h], Vf[:, h // (qh // kvh)].mean(axis=0), rtol=1e-5, atol=1e-6)
    # a wrong head mapping (h % kvh instead of h // group) would fail this
    assert not np.allclose(got[1], Vf[:, 1].mean(axis=0), atol=1e-3)


def test_batched_equals_individual(orc):
    # shape of tests/attention_batched_varlen.rs:36-69 (qh 4, kvh 2, hd 64, lens [1,3,5], ids [0,1,2])
    rng = np.random.default_rng(5)
    qh, kvh, hd, maxL = 4, 2, 64, 8
    K = rng.standard_normal((3, maxL, kvh, hd)).astype(np.float16).view(np.uint16)
    V = rng.standard_normal((3, maxL, kvh, hd)).astype(np.float16).view(np.uint16)
    q = rng.standard_normal((3, qh * hd)).astype(np.float32)
    out = orc.attention_batched(K, V, maxL, kvh, hd, [2, 0, 1], [5, 1, 3], q, qh)
    for b, (sid, L) in enumerate(zip([2, 0, 1], [5, 1, 3])):
        assert np.array_equal(out[b], orc.attention(K, V, maxL, kvh, hd, sid, q[b], qh, L))


# ---------------------------------------------------------------- GEMM / q8_0
def _f16bits(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32).astype(np.float16).view(np.uint16))


def test_gemm_known_answers(orc):
    # tests/gemm_f16xf16_f32.rs:50-52,101-103
    A = _f16bits([[1, 2], [3, 4]]); B = _f16bits([[5, 6], [7, 8]])
    assert np.array_equal(orc.gemm("f16xf16_rowmajor", A, B, 2, 2, 2), [[19, 22], [43, 50]])
    A = _f16bits([[1, 2, 3]]); B = _f16bits([[4, 5], [6, 7], [8, 9]])
    assert np.array_equal(orc.gemm("f16xf16_rowmajor", A, B, 1, 2, 3), [[40, 46]])
    Af = np.array([[1, 2, 3]], dtype=np.float32)
    assert np.array_equal(orc.gemm("f32xf16_rowmajor", Af, B, 1, 2, 3), [[40, 46]])
    # GGUF layout stores the same logical B as B[col*K + k]: the transpose
    Bg = _f16bits(np.array([[4, 5], [6, 7], [8, 9]]).T)
    assert np.array_equal(orc.gemm("f32xf16_gguf", Af, Bg, 1, 2, 3), [[40, 46]])


def test_gemm_vs_float64(orc):
    rng = np.random.default_rng(7)
    M, N, K = 3, 37, 300
    A = rng.standard_normal((M, K)).astype(np.float32)
    Bf = (rng.standard_normal((N, K)) * 0.02).astype(np.float16)
    want = A.astype(np.float64) @ Bf.astype(np.float64).T
    got = orc.gemm("f32xf16_gguf", A, Bf.view(np.uint16), M, N, K)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-6)
    got_rm = orc.gemm("f32xf16_rowmajor", A, np.ascontiguousarray(Bf.T).view(np.uint16), M, N, K)
    assert np.array_equal(got, got_rm)  # same sums, same order, other storage


def _q80_pack(d_f16, qs):
    """d_f16 [nblk] float16, qs [nblk,32] int8 -> bytes [nblk,34]"""
    nblk = qs.shape[0]
    out = np.zeros((nblk, 34), dtype=np.uint8)
    out[:, :2] = d_f16.view(np.uint8).reshape(nblk, 2)
    out[:, 2:] = qs.view(np.uint8)
    return out


def test_q80_reference_fixture(orc):
    # tests/embedding_dequant_cuda.rs:189-206: scale f16(0.25+0.125*row+0.0625*blk), q=((17*row+5*blk+idx)%23)-11
    rows, blks = 3, 2
    for row in range(rows):
        d = np.array([0.25 + 0.125 * row + 0.0625 * b for b in range(blks)], dtype=np.float32).astype(np.float16)
        qs = np.array([[((17 * row + 5 * b + i) % 23) - 11 for i in range(32)] for b in range(blks)], dtype=np.int8)
        got = orc.q80_to_f32(_q80_pack(d, qs), blks * 32)
        want = (d.astype(np.float64)[:, None] * qs.astype(np.float64)).reshape(-1)
        assert np.array_equal(got.astype(np.float64), want)  # products of f16 x int8 are exact in f32


def test_q80_gemm_vs_float64_and_dequant_path(orc):
    rng = np.random.default_rng(11)
    M, N, K = 4, 19, 256
    d = rng.uniform(0.001, 0.01, size=(N, K // 32)).astype(np.float16)
    qs = rng.integers(-127, 128, size=(N, K // 32, 32)).astype(np.int8)
    B = np.stack([_q80_pack(d[n], qs[n]) for n in range(N)])
    A = rng.standard_normal((M, K)).astype(np.float32)
    got = orc.gemm("f32xq80_gguf", A, B, M, N, K)
    W = (d.astype(np.float64)[:, :, None] * qs.astype(np.float64)).reshape(N, K)
    assert np.allclose(got, A.astype(np.float64) @ W.T, rtol=1e-5, atol=1e-6)
    # dequantise with the reference's elementwise kernel semantics, then its f32 GEMM loop: identical bits
    Wf16_exact = orc.q80_to_f32(B.reshape(-1, 34), N * K).reshape(N, K)
    acc = np.zeros((M, N), dtype=np.float32)
    for k in range(K):
        acc = (acc + (A[:, k:k + 1] * Wf16_exact[:, k][None, :]).astype(np.float32)).astype(np.float32)
    assert np.array_equal(got, acc)


# ---------------------------------------------------------------- norm / rope / elementwise
def test_rms_norm_reference_fixtures(orc):
    rows, dim, eps = 2, 8, 1e-5
    x = (np.arange(rows * dim, dtype=np.float32) * 0.25 - 3.0).reshape(rows, dim)
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + eps)
    assert np.allclose(orc.rms_norm(x, eps), want, rtol=1e-6, atol=1e-7)
    x = (np.arange(rows * dim, dtype=np.float32) * 0.125 - 1.0).reshape(rows, dim)
    w = (0.5 + np.arange(dim, dtype=np.float32) * 0.1).astype(np.float32)
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + eps) * w.astype(np.float64)
    assert np.allclose(orc.rms_norm(x, eps, w, 1), want, rtol=1e-6, atol=1e-7)
    w16 = w.astype(np.float16)
    want16 = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + eps) * w16.astype(np.float64)
    assert np.allclose(orc.rms_norm(x, eps, w16.view(np.uint16), 0), want16, rtol=1e-6, atol=1e-7)
    out = np.zeros_like(x)
    assert orc.lib().orc_rms_norm_weighted(orc.ptr(x), orc.ptr(w), orc.ptr(out), rows, dim, eps, 2) == -4


def _f64_rope_adjacent(x, heads, hd, past, base, scale):
    x = x.astype(np.float64).copy()
    rows = x.shape[0]
    for r in range(rows):
        for h in range(heads):
            for i in range(hd // 2):
                th = (past + r) * scale * base ** (-2.0 * i / hd)
                a, b = x[r, h * hd + 2 * i], x[r, h * hd + 2 * i + 1]
                x[r, h * hd + 2 * i] = a * np.cos(th) - b * np.sin(th)
                x[r, h * hd + 2 * i + 1] = a * np.sin(th) + b * np.cos(th)
    return x


def test_rope_adjacent_reference_fixture(orc):
    # tests/rmsnorm_rope.rs:242-264 (rows 1, heads 2, hd 4, past 3) and a 2-row case with past 5
    for rows, past in ((1, 3), (2, 5)):
        x = (np.arange(rows * 8, dtype=np.float32) * 0.1 + 0.5).reshape(rows, 8)
        got = orc.rope(x, 2, 4, past, 10000.0, 1.0, 0)
        assert np.allclose(got, _f64_rope_adjacent(x, 2, 4, past, 10000.0, 1.0), rtol=1e-5, atol=1e-6)


def test_rope_neox_pinned_by_permutation_and_invariants(orc):
    rng = np.random.default_rng(13)
    heads, hd, rows, past = 3, 16, 2, 77
    x = rng.standard_normal((rows, heads * hd)).astype(np.float32)
    # NeoX pair (i, i+hd/2) == adjacent pair (2i, 2i+1) after permuting 2i -> i, 2i+1 -> i+hd/2
    perm = np.zeros(hd, dtype=np.int64)
    perm[: hd // 2] = np.arange(0, hd, 2)
    perm[hd // 2:] = np.arange(1, hd, 2)
    xa = x.reshape(rows, heads, hd)
    x_neox_in = xa[:, :, perm].reshape(rows, heads * hd)          # neox_in[i] = adj[2i], neox_in[i+hd/2] = adj[2i+1]
    got_neox = orc.rope(x_neox_in, heads, hd, past, 1e6, 1.0, 1).reshape(rows, heads, hd)
    got_adj = orc.rope(x, heads, hd, past, 1e6, 1.0, 0).reshape(rows, heads, hd)
    assert np.array_equal(got_neox, got_adj[:, :, perm])
    # position 0 is the identity; rotation preserves each pair's norm
    assert np.array_equal(orc.rope(x, heads, hd, 0, 1e6, 1.0, 1)[0], x[0])
    n_in = x_neox_in.reshape(rows, heads, 2, hd // 2)
    n_out = got_neox.reshape(rows, heads, 2, hd // 2)
    assert np.allclose((n_in ** 2).sum(axis=2), (n_out ** 2).sum(axis=2), rtol=1e-5)
    # rotate_half form: out = x*cos + rotate_half(x)*sin, float64
    i = np.arange(hd // 2)
    for r in range(rows):
        th = (past + r) * 1e6 ** (-2.0 * i / hd)
        c = np.concatenate([np.cos(th), np.cos(th)]); s = np.concatenate([np.sin(th), np.sin(th)])
        xin = x_neox_in.reshape(rows, heads, hd)[r].astype(np.float64)
        rot = np.concatenate([-xin[:, hd // 2:], xin[:, : hd // 2]], axis=1)
        assert np.allclose(got_neox[r], xin * c + rot * s, rtol=1e-4, atol=1e-5)


def test_elementwise_fixtures(orc):
    # closed forms in the style of tests/cuda_elementwise.rs
    n = 513
    g = (np.arange(n, dtype=np.float32) * 0.03 - 7.0).astype(np.float32)
    u = (np.arange(n, dtype=np.float32) * -0.01 + 2.0).astype(np.float32)
    want = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u.astype(np.float64)
    assert np.allclose(orc.swiglu(g, u), want, rtol=1e-6, atol=1e-7)
    assert np.array_equal(orc.residual_add(g, u), g + u)


# ---------------------------------------------------------------- q4 V / compressed cache
def _brute_q4(v_f16):
    v = v_f16.astype(np.float32)
    m = np.float32(np.abs(v).max())
    sc = np.float32(m / np.float32(7)) if m > 0 else np.float32(1) / np.float32(7)
    q = np.clip(np.rint((v / sc).astype(np.float32)), -7, 7).astype(np.int32)
    packed = ((q[0::2] & 15) | ((q[1::2] & 15) << 4)).astype(np.uint8)
    return packed, sc


def test_q4_quantiser_bruteforce(orc):
    rng = np.random.default_rng(17)
    for hd in (64, 128):
        for trial in range(50):
            v = rng.standard_normal(hd).astype(np.float16)
            if trial == 0:
                v[:] = 0
            if trial == 1:
                v = (np.arange(hd) - hd / 2).astype(np.float16)  # exact .5 steps: ties-to-even matters
            packed = np.zeros(hd // 2, dtype=np.uint8); sc = np.zeros(1, dtype=np.float32)
            orc.lib().orc_q4_quantize_row(orc.ptr(np.ascontiguousarray(v.view(np.uint16))), hd, orc.ptr(packed), orc.ptr(sc))
            wp, ws = _brute_q4(v)
            assert np.array_equal(packed, wp) and sc[0] == ws
            # unpack: two's complement nibbles, even dim in the low nibble
            for d in (0, 1, hd - 1):
                nib = (int(packed[d // 2]) >> (4 * (d & 1))) & 15
                assert orc.lib().orc_q4_unpack(int(packed[d // 2]), d & 1, float(sc[0])) == np.float32(nib - 16 if nib >= 8 else nib) * sc[0]


def test_compressed_cache_byte_accounting_literals(orc):
    # tests/attention_parity_cuda_grid.rs:726-843: hd 128, max_seq 16, 1 seq, 2 kv heads -> 8192 / 2048 / 128 bytes
    c = orc.CompressedKV(16, 1, 2, 128, 4, 4)
    assert c.bytes() == (8192, 2048, 128)


def test_compressed_append_evicts_before_overwrite(orc):
    rng = np.random.default_rng(19)
    kvh, hd, W, L = 2, 64, 4, 11
    c = orc.CompressedKV(16, 2, kvh, hd, W, 4)
    ks = rng.standard_normal((L, kvh * hd)).astype(np.float32)
    vs = rng.standard_normal((L, kvh * hd)).astype(np.float32)
    for p in range(L):
        assert c.append(1, p, ks[p], vs[p], 10000.0, 0.0, 0) == 0   # freq_scale 0 -> RoPE is the identity
    k16 = ks.astype(np.float16).view(np.uint16).reshape(L, kvh, hd)
    v16 = vs.astype(np.float16).reshape(L, kvh, hd)
    assert c.seq_map[1] == L and c.seq_map[0] == 0
    assert np.array_equal(c.old_k[1, : L - W], k16[: L - W])
    for t in range(L - W, L):
        assert np.array_equal(c.recent_k[1, t % W], k16[t])
        assert np.array_equal(c.recent_v[1, t % W], v16[t].view(np.uint16))
    for t in range(L - W):
        for h in range(kvh):
            wp, ws = _brute_q4(v16[t, h])
            assert np.array_equal(c.q4_v[1, t, h], wp) and c.q4_scale[1, t, h] == ws
    assert not c.old_k[1, L - W:].any()
    # bulk fill == ordered appends
    c2 = orc.CompressedKV(16, 2, kvh, hd, W, 4)
    c2.bulk_fill(1, k16, v16.view(np.uint16))
    for name in ("old_k", "q4_v", "q4_scale", "recent_k", "recent_v", "seq_map"):
        assert np.array_equal(getattr(c, name), getattr(c2, name)), name
    assert c.append(2, 0, ks[0], vs[0]) == -3 and c.append(0, 16, ks[0], vs[0]) == -5


def test_top_block_selection_bruteforce_and_ties(orc):
    rng = np.random.default_rng(23)
    for n in (1, 5, 64, 200):
        for top in (1, 3, 64):
            s = rng.standard_normal(n).astype(np.float32)
            s[rng.integers(0, n, size=n // 3)] = s[0]        # force ties
            got_b, got_s = orc.select_top_blocks(s, top)
            order = sorted(range(n), key=lambda b: (-float(s[b]), b))[: min(top, n)]
            assert list(got_b) == order
            assert np.array_equal(got_s, s[order])
    s = np.array([np.nan, 1.0, -np.inf, -2e30, 0.5], dtype=np.float32)
    got_b, _ = orc.select_top_blocks(s, 4)
    assert list(got_b) == [1, 4]        # NaN and anything <= -1e30 never enter the list


def test_block_scores_three_orders_agree(orc):
    rng = np.random.default_rng(29)
    for hd in (64, 128):
        kvh, W, bs, L = 2, 8, 16, 8 + 16 * 5 + 7      # last block partial (7 tokens)
        c = orc.CompressedKV(128, 1, kvh, hd, W, bs)
        k16 = rng.standard_normal((L, kvh, hd)).astype(np.float16).view(np.uint16)
        v16 = rng.standard_normal((L, kvh, hd)).astype(np.float16).view(np.uint16)
        c.bulk_fill(0, k16, v16)
        q = rng.standard_normal(hd).astype(np.float32)
        s0 = c.block_scores(0, q, 1, L, 0); s1 = c.block_scores(0, q, 1, L, 1); s2 = c.block_scores(0, q, 1, L, 2)
        assert len(s0) == 6
        kf = k16.view(np.float16).astype(np.float64)[: L - W, 1]
        inv = 0.125 if hd == 64 else 0.08838834764831845
        want = np.array([(kf[b * bs: min((b + 1) * bs, L - W)] @ q.astype(np.float64)).sum()
                         / (min((b + 1) * bs, L - W) - b * bs) * inv for b in range(6)])
        assert np.allclose(s1, want, rtol=1e-12)
        assert np.allclose(s0, want, rtol=1e-4, atol=1e-6) and np.allclose(s2, want, rtol=1e-4, atol=1e-6)


def test_block_select_all_blocks_equals_dense_and_partial_fixture(orc):
    rng = np.random.default_rng(31)
    # tests/attention_parity_cuda_grid.rs:726-843 shape: hd 128, L 16, W 4, bs 4, top 3 (and top >= old_blocks)
    qh, kvh, hd, L, W, bs = 4, 2, 128, 16, 4, 4
    c = orc.CompressedKV(16, 1, kvh, hd, W, bs)
    k = rng.standard_normal((L, kvh, hd)).astype(np.float16)
    v = rng.standard_normal((L, kvh, hd)).astype(np.float16)
    c.bulk_fill(0, k.view(np.uint16), v.view(np.uint16))
    q = rng.standard_normal((qh, hd)).astype(np.float32)
    rc, out, sel, cnt = c.attention(0, q, qh, L, 3)
    assert rc == 0 and list(cnt) == [3] * qh
    # independent float64 evaluation of the same token set with q4-dequantised V
    vq = np.zeros((L, kvh, hd))
    for t in range(L):
        for h in range(kvh):
            if t < L - W:
                p, s = _brute_q4(v[t, h])
                nib = np.stack([p & 15, p >> 4], axis=1).reshape(-1).astype(np.int32)
                nib = np.where(nib >= 8, nib - 16, nib)
                vq[t, h] = (nib.astype(np.float32) * s).astype(np.float16).astype(np.float64)
            else:
                vq[t, h] = v[t, h].astype(np.float64)
    inv = 0.08838834764831845
    for h in range(qh):
        kvhh = h // (qh // kvh)
        toks = [t for b in sel[h][:3] for t in range(b * bs, (b + 1) * bs)] + list(range(L - W, L))
        s = np.array([k[t, kvhh].astype(np.float64) @ q[h].astype(np.float64) for t in toks]) * inv
        p = np.exp(s - s.max()); p /= p.sum()
        want = sum(pi * vq[t, kvhh] for pi, t in zip(p, toks))
        assert np.allclose(out[h * hd:(h + 1) * hd], want, rtol=1e-4, atol=1e-5)
    # top >= old_blocks: every token attended -> equals dense attention over dequantised V (float64)
    rc, out_all, _, cnt = c.attention(0, q, qh, L, 64)
    assert rc == 0 and list(cnt) == [3] * qh
    for h in range(qh):
        kvhh = h // (qh // kvh)
        s = (k[:, kvhh].astype(np.float64) @ q[h].astype(np.float64)) * inv
        p = np.exp(s - s.max()); p /= p.sum()
        assert np.allclose(out_all[h * hd:(h + 1) * hd], p @ vq[:, kvhh], rtol=1e-4, atol=1e-5)
    # partial old block (L 5, W 4, bs 32, top 8): tests/attention_parity_cuda_grid.rs:608-723
    rc, out5, sel5, cnt5 = c.attention(0, q, qh, 5, 8, recent_window=4, block_size=32)
    assert rc == 0 and list(cnt5) == [1] * qh and all(sel5[:, 0] == 0)
    # error codes of the argument checks
    assert c.attention(0, q, qh, 0, 3)[0] == -3 and c.attention(0, q, 3, L, 3)[0] == -4
    assert c.attention(0, q, qh, L, 65)[0] == -6 and c.attention(0, q, qh, L, 0)[0] == -6


# ---- old V in groups of 32 with an f16 scale and an f16 minimum (the benchmark configuration's V format; the reference
# has none, so the definition in oracle.c is the contract and these are its pins)
def _brute_q4g32(v_f16):
    """float64 / numpy restatement: per group d = f16((max - min) / 15), m = f16(min), q = rint((v - m) / d) in 0..15."""
    v = v_f16.astype(np.float32).reshape(-1, 32)
    mn, mx = v.min(axis=1), v.max(axis=1)
    d16 = ((mx - mn) / np.float32(15)).astype(np.float16); m16 = mn.astype(np.float16)
    d, m = d16.astype(np.float32), m16.astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(d[:, None] > 0, np.clip(np.rint(((v - m[:, None]) / d[:, None]).astype(np.float32)), 0, 15), 0).astype(np.uint8)
    q = q.reshape(-1)
    packed = (q[0::2] | (q[1::2] << 4)).astype(np.uint8)
    dm = d16.view(np.uint16).astype(np.uint32) | (m16.view(np.uint16).astype(np.uint32) << 16)
    return packed, dm, q, d, m


def _q4g32(orc, v_f16):
    hd = v_f16.size
    packed = np.zeros(hd // 2, dtype=np.uint8); dm = np.zeros(hd // 32, dtype=np.uint32)
    orc.lib().orc_q4g32_quantize_row(orc.ptr(np.ascontiguousarray(v_f16.view(np.uint16))), hd, orc.ptr(packed), orc.ptr(dm))
    deq = np.array([orc.lib().orc_q4g32_unpack(int(packed[i // 2]), i & 1, int(dm[i // 32])) for i in range(hd)], dtype=np.float32)
    return packed, dm, deq


def test_q4_group32_closed_forms(orc):
    hd = 128
    # (1) values on an exact grid min + k * step (min, step and 15 * step exact in f16): the round trip is exact, the
    # nibble is k, even dimensions sit in the low nibble, the word is bits(step) | bits(min) << 16
    ks = np.tile(np.array([0, 15, 3, 12, 7, 8, 1, 14, 5, 10, 2, 13, 6, 9, 4, 11] * 2), hd // 32)
    v = (np.float32(-2.0) + np.float32(0.25) * ks).astype(np.float16)
    packed, dm, deq = _q4g32(orc, v)
    assert np.array_equal(deq, v.astype(np.float32))
    assert np.array_equal(packed, (ks[0::2] | (ks[1::2] << 4)).astype(np.uint8))
    want_dm = int(np.float16(0.25).view(np.uint16)) | (int(np.float16(-2.0).view(np.uint16)) << 16)
    assert all(int(w) == want_dm for w in dm)
    # (2) a constant group: scale 0, every nibble 0, every value the constant itself; an all-zero row likewise
    v = np.full(hd, np.float16(1.25)); v[32:64] = np.float16(-0.375); v[64:] = 0
    packed, dm, deq = _q4g32(orc, v)
    assert not packed.any() and np.array_equal(deq, v.astype(np.float32))
    assert [int(w) & 0xffff for w in dm] == [0, 0, 0, 0]
    # (3) the two ends of a group map to nibbles 0 and 15, and every value is within half a step (plus the rounding
    # of the stored minimum and scale) of what went in
    rng = np.random.default_rng(23)
    for trial in range(40):
        v = (rng.standard_normal(hd) * rng.uniform(0.01, 30.0)).astype(np.float16)
        packed, dm, deq = _q4g32(orc, v)
        wp, wdm, q, d, m = _brute_q4g32(v)
        assert np.array_equal(packed, wp) and np.array_equal(dm, wdm)            # independent restatement, same bytes
        vf = v.astype(np.float32).reshape(-1, 32); qg = q.reshape(-1, 32)
        for g in range(hd // 32):
            assert qg[g, vf[g].argmin()] == 0 and qg[g, vf[g].argmax()] >= 14
            bound = 0.5 * d[g] * (1 + 2.0 ** -9) + abs(m[g] - vf[g].min()) + 15 * abs(d[g] - (vf[g].max() - vf[g].min()) / 15) + 1e-7
            assert np.abs(deq.reshape(-1, 32)[g] - vf[g]).max() <= bound
        # value = fmaf(q, d, m): one rounding of the exact q * d + m
        exact = q.astype(np.float64) * np.repeat(d, 32).astype(np.float64) + np.repeat(m, 32).astype(np.float64)
        assert np.array_equal(deq, exact.astype(np.float32))


def test_compressed_cache_group32_bytes_appends_and_attention(orc):
    rng = np.random.default_rng(29)
    qh, kvh, hd, L, W, bs = 4, 2, 128, 24, 4, 4
    c = orc.CompressedKV(32, 1, kvh, hd, W, bs, v_format=1)
    # 16 B of scale | min words per (token, head) beside 64 B of nibbles: 80 B against the reference format's 68
    assert c.bytes() == (32 * kvh * hd * 2, 32 * kvh * hd // 2, 32 * kvh * (hd // 32) * 4)
    k = rng.standard_normal((L, kvh, hd)).astype(np.float16)
    v = (2.0 * rng.standard_normal((L, kvh, hd))).astype(np.float16)
    for p in range(L):
        assert c.append(0, p, k[p].astype(np.float32).reshape(-1), v[p].astype(np.float32).reshape(-1), 1e4, 0.0, 0) == 0
    for t in range(L - W):
        for h in range(kvh):
            wp, wdm, _, _, _ = _brute_q4g32(v[t, h])
            assert np.array_equal(c.q4_v[0, t, h], wp) and np.array_equal(c.q4_dm[0, t, h], wdm)
    c2 = orc.CompressedKV(32, 1, kvh, hd, W, bs, v_format=1)
    c2.bulk_fill(0, k.view(np.uint16), v.view(np.uint16))
    for name in ("old_k", "q4_v", "q4_dm", "recent_k", "recent_v", "seq_map"):
        assert np.array_equal(getattr(c, name), getattr(c2, name)), name
    # attention over everything (top >= old blocks) = float64 softmax over the dequantised V
    q = rng.standard_normal((qh, hd)).astype(np.float32)
    rc, out, sel, cnt = c.attention(0, q, qh, L, 64, score_order=0)
    assert rc == 0 and list(cnt) == [5] * qh
    vq = v.astype(np.float64).copy()
    for t in range(L - W):
        for h in range(kvh):
            _, _, qn, d, m = _brute_q4g32(v[t, h])
            vq[t, h] = (qn.astype(np.float64) * np.repeat(d, 32) + np.repeat(m, 32)).astype(np.float32)
    for h in range(qh):
        kvhh = h // (qh // kvh)
        s = (k[:, kvhh].astype(np.float64) @ q[h].astype(np.float64)) * 0.08838834764831845
        p = np.exp(s - s.max()); p /= p.sum()
        assert np.allclose(out[h * hd:(h + 1) * hd], p @ vq[:, kvhh], rtol=1e-4, atol=1e-5)
    # V rows that the format holds exactly: the compressed cache and a dense f16 cache give the same attention
    vg = (np.float32(-1.0) + np.float32(0.125) * rng.integers(0, 16, size=(L, kvh, hd))).astype(np.float16)
    vg[:, :, 0::32] = np.float16(-1.0); vg[:, :, 1::32] = np.float16(0.875)          # every group spans the whole grid
    c3 = orc.CompressedKV(32, 1, kvh, hd, W, bs, v_format=1)
    c3.bulk_fill(0, k.view(np.uint16), vg.view(np.uint16))
    rc, out3, sel3, _ = c3.attention(0, q, qh, L, 3, score_order=0)
    K = np.zeros((1, 32, kvh, hd), dtype=np.uint16); V = np.zeros_like(K)
    K[0, :L] = k.view(np.uint16); V[0, :L] = vg.view(np.uint16)
    rc2, outd, seld, _ = orc.dense_block_select(K, V, 32, kvh, hd, 0, q, qh, L, W, bs, 3, score_order=0)
    assert rc == 0 and rc2 == 0 and np.array_equal(sel3, seld)
    assert np.allclose(out3, outd, rtol=1e-6, atol=1e-7)


def test_dense_backed_block_select_matches_dense_when_all_selected(orc):
    # property of tests/attention_parity_cuda_grid.rs:182-486
    rng = np.random.default_rng(37)
    qh, kvh, hd, L, W, bs = 8, 2, 64, 40, 8, 8
    K = rng.standard_normal((1, 64, kvh, hd)).astype(np.float16).view(np.uint16)
    V = rng.standard_normal((1, 64, kvh, hd)).astype(np.float16).view(np.uint16)
    q = rng.standard_normal((qh, hd)).astype(np.float32)
    rc, out, sel, cnt = orc.dense_block_select(K, V, 64, kvh, hd, 0, q, qh, L, W, bs, 64)
    assert rc == 0 and list(cnt) == [4] * qh
    dense = orc.attention(K, V, 64, kvh, hd, 0, q, qh, L)
    assert np.allclose(out, dense, rtol=1e-4, atol=1e-5)


def test_debug_select_host_twin(orc):
    rng = np.random.default_rng(41)
    kvh, hd, W, bs, L = 2, 64, 8, 4, 8 + 4 * 9 + 2
    c = orc.CompressedKV(64, 1, kvh, hd, W, bs)
    k16 = rng.standard_normal((L, kvh, hd)).astype(np.float16)
    c.bulk_fill(0, k16.view(np.uint16), k16.view(np.uint16))
    q0 = rng.standard_normal(hd).astype(np.float32)
    rc, blocks, scores, start, end, total = c.debug_select(0, q0, L, 3)
    assert rc == 0 and total == 10 and len(blocks) == 3
    kf = k16.astype(np.float64)[: L - W, 0]
    want = [(kf[b * bs: min((b + 1) * bs, L - W)] @ q0.astype(np.float64)).sum()
            / (min((b + 1) * bs, L - W) - b * bs) * 0.125 for b in range(10)]
    order = sorted(range(10), key=lambda b: (-want[b], b))[:3]
    assert list(blocks) == order
    assert list(start) == [b * bs for b in order] and list(end) == [min((b + 1) * bs, L - W) for b in order]
    assert np.allclose(scores, [want[b] for b in order], rtol=1e-4)


# ---------------------------------------------------------------- sampling
def test_greedy_reference_literals(orc):
    # src/sampling.rs:171-175, :196-207, :243-250
    assert orc.sample_greedy([0.1, -0.2, 5.0, 1.0]) == 2
    assert orc.greedy_topk1([0.0, 5.0, 1.0]) == 1
    assert orc.greedy_topk1([np.nan, -1.0, 3.0]) == 2
    assert orc.greedy_topk1([2.0, 2.0, 1.0]) == 0       # stable order: lowest index wins ties
    assert orc.greedy_topk1([-np.inf, -np.inf]) == 0


# ---------------------------------------------------------------- layer / model
def make_toy_model(rng, qkv_bias, rope_layout, n_layers=2, d_model=64, q_heads=4, kv_heads=2, ffn=96, vocab=50):
    hd = d_model // q_heads
    kv_dim = kv_heads * hd
    cfg = dict(n_layers=n_layers, d_model=d_model, q_heads=q_heads, kv_heads=kv_heads, head_dim=hd, ffn=ffn,
               vocab=vocab, rms_eps=1e-5, rope_base=10000.0, rope_scale=1.0, rope_layout=rope_layout,
               qkv_bias=qkv_bias)

    def w(n, k, s=0.2):
        return np.ascontiguousarray((rng.standard_normal((n, k)) * s).astype(np.float16).view(np.uint16))

    W = dict(
        wq=[w(d_model, d_model) for _ in range(n_layers)], wk=[w(kv_dim, d_model) for _ in range(n_layers)],
        wv=[w(kv_dim, d_model) for _ in range(n_layers)], wo=[w(d_model, d_model) for _ in range(n_layers)],
        wgate=[w(ffn, d_model) for _ in range(n_layers)], wup=[w(ffn, d_model) for _ in range(n_layers)],
        wdown=[w(d_model, ffn) for _ in range(n_layers)],
        attn_norm=[(1 + 0.1 * rng.standard_normal(d_model)).astype(np.float32) for _ in range(n_layers)],
        ffn_norm=[(1 + 0.1 * rng.standard_normal(d_model)).astype(np.float32) for _ in range(n_layers)],
        out_norm=(1 + 0.1 * rng.standard_normal(d_model)).astype(np.float32),
        lm_head=w(vocab, d_model), tok_emb=w(vocab, d_model, 1.0))
    if qkv_bias:
        W["bq"] = [(0.1 * rng.standard_normal(d_model)).astype(np.float32) for _ in range(n_layers)]
        W["bk"] = [(0.1 * rng.standard_normal(kv_dim)).astype(np.float32) for _ in range(n_layers)]
        W["bv"] = [(0.1 * rng.standard_normal(kv_dim)).astype(np.float32) for _ in range(n_layers)]
    return cfg, W


def f64_model_logits(cfg, W, ids, kv_through_f16=True, want_hidden=False):
    """Independent float64 restatement of the decoder (full-sequence causal attention), last-token logits.
    kv_through_f16: K and V pass through the f16 cache (the token-by-token path); False = the packed prefill, whose
    attention reads the f32 rows."""
    f = lambda a: a.view(np.float16).astype(np.float64)
    D, H, KVH, hd = cfg["d_model"], cfg["q_heads"], cfg["kv_heads"], cfg["head_dim"]
    T = len(ids)
    x = f(W["tok_emb"])[ids]

    def norm(x, w):
        return x / np.sqrt((x ** 2).mean(-1, keepdims=True) + cfg["rms_eps"]) * w.astype(np.float64)

    def rope(t, nh):
        t = t.reshape(T, nh, hd).copy()
        pos = np.arange(T)[:, None]
        i = np.arange(hd // 2)[None, :]
        th = pos * cfg["rope_base"] ** (-2.0 * i / hd)
        c, s = np.cos(th)[:, None, :], np.sin(th)[:, None, :]
        if cfg["rope_layout"] == 0:
            a, b = t[..., 0::2].copy(), t[..., 1::2].copy()
            t[..., 0::2], t[..., 1::2] = a * c - b * s, a * s + b * c
        else:
            a, b = t[..., : hd // 2].copy(), t[..., hd // 2:].copy()
            t[..., : hd // 2], t[..., hd // 2:] = a * c - b * s, a * s + b * c
        return t
    h16 = (lambda a: a.astype(np.float16).astype(np.float64)) if kv_through_f16 else (lambda a: a)
    for l in range(cfg["n_layers"]):
        xn = norm(x, W["attn_norm"][l])
        q = xn @ f(W["wq"][l]).T; k = xn @ f(W["wk"][l]).T; v = xn @ f(W["wv"][l]).T
        if cfg["qkv_bias"]:
            q = q + W["bq"][l]; k = k + W["bk"][l]; v = v + W["bv"][l]
        q = rope(q, H); k = h16(rope(k, KVH)); v = h16(v.reshape(T, KVH, hd))
        ctx = np.zeros((T, H, hd))
        for hh in range(H):
            s = (q[:, hh] @ k[:, hh // (H // KVH)].T) / np.sqrt(hd)
            s = np.where(np.tril(np.ones((T, T))) > 0, s, -np.inf)
            p = np.exp(s - s.max(-1, keepdims=True)); p /= p.sum(-1, keepdims=True)
            ctx[:, hh] = p @ v[:, hh // (H // KVH)]
        x = x + ctx.reshape(T, D) @ f(W["wo"][l]).T
        xn = norm(x, W["ffn_norm"][l])
        g = xn @ f(W["wgate"][l]).T; u = xn @ f(W["wup"][l]).T
        x = x + (g / (1 + np.exp(-g)) * u) @ f(W["wdown"][l]).T
    if want_hidden:
        return x
    return norm(x[-1:], W["out_norm"]) @ f(W["lm_head"]).T


@pytest.mark.parametrize("qkv_bias,layout", [(False, 0), (True, 1)])
def test_model_decode_vs_float64(orc, qkv_bias, layout):
    rng = np.random.default_rng(43 + layout)
    cfg, W = make_toy_model(rng, qkv_bias, layout)
    m = orc.Model(cfg, W)
    m.alloc_kv(16, 1)
    ids = [3, 17, 42, 8, 8, 29]
    for pos, t in enumerate(ids):
        hidden = m.token_forward(0, pos, t)
    got = m.logits(hidden)
    want = f64_model_logits(cfg, W, np.array(ids))[0]
    assert np.allclose(got, want, rtol=2e-3, atol=2e-3), np.abs(got - want).max()
    assert int(np.argmax(got)) == int(np.argmax(want))
    # greedy decode continues deterministically and reports top-2 gaps
    m.alloc_kv(16, 1)
    out_ids, gaps = m.decode_greedy(0, ids, 4)
    assert list(out_ids[: len(ids)]) == ids and out_ids[len(ids)] == int(np.argmax(want))
    assert (gaps >= 0).all()


@pytest.mark.parametrize("qkv_bias,layout", [(False, 0), (True, 1)])
def test_packed_prefill_forward_vs_float64_and_token_by_token(orc, qkv_bias, layout):
    # src/infer/forward.rs:2153-2600: the packed prefill's attention reads the f32 K / V rows, the f16 cache is written on
    # the side.  The float64 restatement without the f16 round trip must fit tightly, the one with it must not (the bound
    # tells the two apart); the token-by-token path agrees within the reference's own whole-model tolerance
    # (tests/forward_parity_toy.rs:389); a batch of prompts equals each prompt alone; and the cache the prefill leaves
    # serves the decode that follows.
    rng = np.random.default_rng(53 + layout)
    cfg, W = make_toy_model(rng, qkv_bias, layout, n_layers=3, d_model=256, ffn=160)      # head_dim 64: the packed attention takes 64 or 128
    prompts = [[3, 17, 42, 8, 8, 29, 11, 2, 40], [5], [7, 7, 30, 1]]
    m = orc.Model(cfg, W)
    m.alloc_kv(16, 3)
    rows = m.prefill_forward([2, 0, 1], prompts)
    off = np.concatenate([[0], np.cumsum([len(p) for p in prompts])])
    for i, p in enumerate(prompts):
        got = rows[off[i]:off[i + 1]]
        want = f64_model_logits(cfg, W, np.array(p), kv_through_f16=False, want_hidden=True)
        rounded = f64_model_logits(cfg, W, np.array(p), kv_through_f16=True, want_hidden=True)
        scale = np.abs(want).max()
        assert np.abs(got - want).max() <= 2e-5 * scale, (i, np.abs(got - want).max() / scale)
        if len(p) > 1:      # one token: softmax over one key, the rounding of K has no effect and that of V is below the bound
            assert np.abs(got - rounded).max() > 2e-5 * scale, (i, np.abs(got - rounded).max() / scale)
        alone = orc.Model(cfg, W)
        alone.alloc_kv(16, 1)
        assert np.array_equal(alone.prefill_forward([0], [p]).view(np.uint32), got.view(np.uint32))
        tok = orc.Model(cfg, W)
        tok.alloc_kv(16, 1)
        for pos, t in enumerate(p):
            h = tok.token_forward(0, pos, t)
        assert np.abs(got[-1] - h).max() <= 5e-3 * max(1.0, np.abs(h).max())
        # layer 0 sees the same rows in both paths: its cache entries are the same bits
        Kp, Vp = alone.kv_views(); Kt, Vt = tok.kv_views()
        assert np.array_equal(Kp[0, :len(p)], Kt[0, :len(p)]) and np.array_equal(Vp[0, :len(p)], Vt[0, :len(p)])
    # the decode that follows a prefill continues from its cache
    ids, _ = m.decode_greedy(2, [int(np.argmax(m.logits(rows[off[1] - 1])))], 3, start_pos=len(prompts[0]))
    assert len(ids) == 4


def test_layer_single_token_context_is_v(orc):
    # L = 1 => attention context equals V (tests/forward_parity_toy.rs:121-386 relies on the same fact)
    rng = np.random.default_rng(47)
    cfg, W = make_toy_model(rng, False, 0, n_layers=1)
    m = orc.Model(cfg, W)
    m.alloc_kv(4, 1)
    x = rng.standard_normal(cfg["d_model"]).astype(np.float32)
    out = m.layer_forward(0, 0, 0, x)
    f = lambda a: a.view(np.float16).astype(np.float64)
    x64 = x.astype(np.float64)
    nrm = lambda z, w: z / np.sqrt((z ** 2).mean() + cfg["rms_eps"]) * w
    xn = nrm(x64, W["attn_norm"][0])
    v = (xn @ f(W["wv"][0]).T).astype(np.float16).astype(np.float64).reshape(cfg["kv_heads"], cfg["head_dim"])
    ctx = np.repeat(v, cfg["q_heads"] // cfg["kv_heads"], axis=0).reshape(-1)
    x1 = x64 + ctx @ f(W["wo"][0]).T
    xn = nrm(x1, W["ffn_norm"][0])
    g = xn @ f(W["wgate"][0]).T; u = xn @ f(W["wup"][0]).T
    want = x1 + (g / (1 + np.exp(-g)) * u) @ f(W["wdown"][0]).T
    assert np.allclose(out, want, rtol=2e-3, atol=2e-3)


# ---------------------------------------------------------------- packed varlen prefill attention
def _f64_prefill(q, k, v, q_lens, kv_lens, qh, kvh, hd):
    out = np.zeros(q.shape, dtype=np.float64)
    qo = np.concatenate([[0], np.cumsum(q_lens)[:-1]]); ko = np.concatenate([[0], np.cumsum(kv_lens)[:-1]])
    g = qh // kvh
    for b in range(len(q_lens)):
        for qi in range(q_lens[b]):
            end = kv_lens[b] - q_lens[b] + qi
            for h in range(qh):
                kk = k[ko[b]:ko[b] + end + 1, h // g].astype(np.float64)
                vv = v[ko[b]:ko[b] + end + 1, h // g].astype(np.float64)
                s = kk @ q[qo[b] + qi, h].astype(np.float64) / np.sqrt(hd)
                p = np.exp(s - s.max()); p /= p.sum()
                out[qo[b] + qi, h] = p @ vv
    return out


def _modular_fixture(n, spec):
    i = np.arange(n, dtype=np.int64)
    return ((i * spec["mul"] % spec["mod"]).astype(np.float32) * np.float32(spec["scale"]) + np.float32(spec["offset"])).astype(np.float32)


def test_prefill_varlen_reference_fixture_vs_float64(orc):
    import json, os
    g = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_literals.json")))["attention_prefill_varlen"]
    ql = [s["query_len"] for s in g["sequences"]]; kl = [s["kv_len"] for s in g["sequences"]]
    qh, kvh = g["q_heads"], g["kv_heads"]
    for hd in g["head_dims"]:
        q = _modular_fixture(sum(ql) * qh * hd, g["q"]).reshape(sum(ql), qh, hd)
        k = _modular_fixture(sum(kl) * kvh * hd, g["k"]).reshape(sum(kl), kvh, hd)
        v = _modular_fixture(sum(kl) * kvh * hd, g["v"]).reshape(sum(kl), kvh, hd)
        rc, got = orc.attention_prefill(q, k, v, ql, kl, qh, kvh, hd)
        assert rc == 0
        assert np.allclose(got, _f64_prefill(q, k, v, ql, kl, qh, kvh, hd), rtol=1e-5, atol=1e-6)


def test_prefill_varlen_invariants_and_codes(orc):
    rng = np.random.default_rng(5)
    qh, kvh, hd = 6, 2, 64
    ql, kl = [4, 1, 7], [4, 9, 10]          # full prefill, one-token decode, chunked prefill (3 cached tokens)
    q = rng.standard_normal((sum(ql), qh, hd)).astype(np.float32)
    k = rng.standard_normal((sum(kl), kvh, hd)).astype(np.float16).astype(np.float32)
    v = rng.standard_normal((sum(kl), kvh, hd)).astype(np.float16).astype(np.float32)
    rc, got = orc.attention_prefill(q, k, v, ql, kl, qh, kvh, hd)
    assert rc == 0
    assert np.allclose(got, _f64_prefill(q, k, v, ql, kl, qh, kvh, hd), rtol=1e-5, atol=1e-6)
    # the first query of a full prefill sees one key: its output is that V row, exactly
    assert np.array_equal(got[0], np.repeat(v[0], qh // kvh, axis=0))
    # a one-token sequence is last-token attention over its keys (the decode oracle on the same f16-exact values)
    K16 = np.ascontiguousarray(k[4:13].astype(np.float16).view(np.uint16)[None]); V16 = np.ascontiguousarray(v[4:13].astype(np.float16).view(np.uint16)[None])
    want = orc.attention(K16, V16, 9, kvh, hd, 0, q[4].reshape(-1), qh, 9)
    assert np.allclose(got[4].reshape(-1), want, rtol=1e-6, atol=1e-7)
    # the batch is the sequences one by one
    rc1, solo = orc.attention_prefill(q[5:], k[13:], v[13:], [7], [10], qh, kvh, hd)
    assert rc1 == 0 and np.array_equal(solo, got[5:])
    # argument checks of cuda/kernels.cu:4849-4887
    assert orc.attention_prefill(q, k, v, ql, kl, qh, kvh, 32)[0] == -9
    assert orc.attention_prefill(q, k, v, ql, kl, 5, 2, hd)[0] == -3
    assert orc.attention_prefill(q, k, v, [4, 1, 11], kl, qh, kvh, hd)[0] == -8      # query longer than its keys
    assert orc.attention_prefill(q, k, v, [4, 0, 7], kl, qh, kvh, hd)[0] == -8
    assert orc.attention_prefill(q, k, v, [4, 1, 7], [4, 9, 8193], qh, kvh, hd)[0] == -8
