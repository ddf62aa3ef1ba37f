"""Parity of the HIP path against the CPU oracle, called through the C-ABI on a real GPU."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    from gpu_common import Dev
    d = Dev()
    yield d
    d.sync()


from gpu_common import RTOL, close, f16bits, m40  # noqa: E402


# ------------------------------------------------------------------ elementwise
def test_rms_norm(dev, orc):
    rng = np.random.default_rng(0)
    for rows, dim in ((2, 8), (1, 2048), (8, 2048), (3, 4096), (2, 37)):
        x = rng.standard_normal((rows, dim)).astype(np.float32)
        if (rows, dim) == (2, 8):
            x = (np.arange(16, dtype=np.float32) * 0.25 - 3.0).reshape(2, 8)   # tests/rmsnorm_rope.rs:85-89
        dx, dy = dev.up(x), dev.zeros(x.nbytes)
        dev.call("m40llm_rms_norm_f32", dx.ptr, dy.ptr, rows, dim, 1e-5)
        close(dy.download(np.float32, x.shape), orc.rms_norm(x, 1e-5), 1e-4, 1e-5)
        w = (0.5 + 0.1 * rng.standard_normal(dim)).astype(np.float32)
        for wd, wbits in ((1, w), (0, w.astype(np.float16).view(np.uint16))):
            dw = dev.up(wbits)
            dev.call("m40llm_rms_norm_f32_weighted", dx.ptr, dw.ptr, dy.ptr, rows, dim, 1e-5, wd)
            close(dy.download(np.float32, x.shape), orc.rms_norm(x, 1e-5, wbits, wd), 1e-4, 1e-5)
    dev.call("m40llm_rms_norm_f32_weighted_async", dx.ptr, dw.ptr, dy.ptr, 1, 8, 1e-5, 2, expect=-4)
    dev.call("m40llm_rms_norm_f32_async", None, dy.ptr, 1, 8, 1e-5, expect=-1)
    dev.call("m40llm_rms_norm_f32_async", dx.ptr, dy.ptr, 1, 0, 1e-5, expect=-1)


@pytest.mark.parametrize("layout", [0, 1])
def test_rope(dev, orc, layout):
    rng = np.random.default_rng(1)
    for rows, heads, hd, past, base in ((1, 2, 4, 3, 1e4), (2, 2, 4, 5, 1e4), (1, 32, 64, 159, 1e4),
                                        (8, 16, 128, 4100, 1e6), (3, 4, 128, 32767, 1e6)):
        x = rng.standard_normal((rows, heads * hd)).astype(np.float32)
        dx = dev.up(x)
        dev.call("m40llm_rope_f32_inplace_layout_async", dx.ptr, rows, heads, hd, past, base, 1.0, layout)
        dev.sync()
        close(dx.download(np.float32, x.shape), orc.rope(x, heads, hd, past, base, 1.0, layout), 1e-4, 1e-4)
        # q&k form
        dq, dk = dev.up(x), dev.up(x * 2)
        dev.call("m40llm_rope_f32_layout_async", dq.ptr, dk.ptr, rows, heads, hd, past, base, 1.0, layout)
        dev.sync()
        close(dk.download(np.float32, x.shape), orc.rope(x * 2, heads, hd, past, base, 1.0, layout), 1e-4, 1e-4)
        # position read from the device
        dpos = dev.up(np.array([past], dtype=np.uint32))
        dx2 = dev.up(x)
        dev.call("m40llm_rope_f32_inplace_position_dev_layout_async", dx2.ptr, rows, heads, hd, dpos.ptr, base, 1.0, layout)
        dev.sync()
        assert np.array_equal(dx2.download(np.float32, x.shape), dx.download(np.float32, x.shape))
    dev.call("m40llm_rope_f32_inplace_layout_async", dx.ptr, 1, 2, 5, 0, 1e4, 1.0, layout, expect=-2)
    dev.call("m40llm_rope_f32_inplace_layout_async", dx.ptr, 1, 0, 4, 0, 1e4, 1.0, layout, expect=-1)


def test_swiglu_residual_casts(dev, orc):
    rng = np.random.default_rng(2)
    n = 5632 * 3 + 1
    g = (rng.standard_normal(n) * 4).astype(np.float32); u = rng.standard_normal(n).astype(np.float32)
    dg, du, do = dev.up(g), dev.up(u), dev.zeros(n * 4)
    dev.call("m40llm_swiglu_f32", dg.ptr, du.ptr, do.ptr, n)
    close(do.download(np.float32, (n,)), orc.swiglu(g, u), 1e-5, 1e-6)        # tests/cuda_elementwise.rs: 1e-5
    dev.call("m40llm_residual_add_f32", dg.ptr, du.ptr, do.ptr, n)
    assert np.array_equal(do.download(np.float32, (n,)), g + u)
    dev.call("m40llm_swiglu_f32_async", dg.ptr, du.ptr, do.ptr, 0)
    dev.call("m40llm_residual_add_f32_async", None, du.ptr, do.ptr, 4, expect=-1)
    h = rng.standard_normal(1000).astype(np.float16)
    dh, df = dev.up(h.view(np.uint16)), dev.zeros(4000)
    dev.call("m40llm_f16_to_f32", dh.ptr, df.ptr, 1000)
    assert np.array_equal(df.download(np.float32, (1000,)), h.astype(np.float32))


def _q80_pack(d_f16, qs):
    nblk = qs.shape[0]
    out = np.zeros((nblk, 34), dtype=np.uint8)
    out[:, :2] = d_f16.view(np.uint8).reshape(nblk, 2)
    out[:, 2:] = qs.view(np.uint8)
    return out


def test_q80_dequant_reference_fixture(dev, orc):
    rows, blks = 3, 2     # tests/embedding_dequant_cuda.rs:189-206
    for row in range(rows):
        d = np.array([0.25 + 0.125 * row + 0.0625 * b for b in range(blks)], dtype=np.float32).astype(np.float16)
        qs = np.array([[((17 * row + 5 * b + i) % 23) - 11 for i in range(32)] for b in range(blks)], dtype=np.int8)
        blob = _q80_pack(d, qs)
        din, dout = dev.up(blob), dev.zeros(blks * 32 * 4)
        dev.call("m40llm_q80_to_f32", din.ptr, dout.ptr, blks * 32)
        assert np.array_equal(dout.download(np.float32, (blks * 32,)), orc.q80_to_f32(blob, blks * 32))


# ------------------------------------------------------------------ KV append
def test_kv_append_cast_bit_exact(dev, orc):
    # fixtures of tests/kv_f32_to_f16_append.rs (odd element count included)
    for heads, hd in ((1, 3), (2, 8), (4, 64)):
        elems = heads * hd
        kv = m40.KVCache(dev.ctx, 4, 2, heads, hd)
        i = np.arange(elems, dtype=np.float32)
        toks = [((i + 0.25).astype(np.float32), (100 + i + 0.5).astype(np.float32)),
                ((-10 + 0.125 * i).astype(np.float32), (np.float32(np.pi) + 0.25 * i).astype(np.float32))]
        for t, (k, v) in enumerate(toks):
            dk, dv = dev.up(k), dev.up(v)
            dev.call("m40llm_kvcache_append_token_f32", kv.h, 1, dk.ptr, dv.ptr)
            gk, gv = kv.read_token(1, t)
            assert np.array_equal(gk, k.astype(np.float16).view(np.uint16))
            assert np.array_equal(gv, v.astype(np.float16).view(np.uint16))
        gk, _ = kv.read_token(0, 0)
        assert not gk.any()
        # cache full after max_seq_len appends -> -4; reset -> position 0 again
        for _ in range(2):
            dev.call("m40llm_kvcache_append_token_f32_async", kv.h, 1, dk.ptr, dv.ptr)
        dev.call("m40llm_kvcache_append_token_f32_async", kv.h, 1, dk.ptr, dv.ptr, expect=-4)
        dev.call("m40llm_kvcache_append_token_f32_async", kv.h, 2, dk.ptr, dv.ptr, expect=-2)
        dev.call("m40llm_kvcache_reset", kv.h)
        dev.call("m40llm_kvcache_append_token_f32", kv.h, 1, dk.ptr, dv.ptr)
        gk, _ = kv.read_token(1, 0)
        assert np.array_equal(gk, toks[1][0].astype(np.float16).view(np.uint16))
        # f16 D2D append
        kv2 = m40.KVCache(dev.ctx, 4, 1, heads, hd)
        hk = dev.up(toks[0][0].astype(np.float16).view(np.uint16)); hv = dev.up(toks[0][1].astype(np.float16).view(np.uint16))
        dev.call("m40llm_kvcache_append_token", kv2.h, 0, hk.ptr, hv.ptr)
        gk, gv = kv2.read_token(0, 0)
        assert np.array_equal(gv, toks[0][1].astype(np.float16).view(np.uint16))


@pytest.mark.parametrize("layout", [0, 1])
def test_kv_append_rope_k_fused_equals_standalone(dev, orc, layout):
    # tests/kv_f32_to_f16_append.rs:297-384: fused RoPE-K append must be bit-identical (u16) to
    # standalone rope_f32_inplace + cast append on the same device
    rng = np.random.default_rng(3)
    for heads, hd, base in ((4, 64, 1e4), (2, 128, 1e6)):
        elems = heads * hd
        kv_a = m40.KVCache(dev.ctx, 64, 1, heads, hd)
        kv_b = m40.KVCache(dev.ctx, 64, 1, heads, hd)
        kv_c = m40.KVCache(dev.ctx, 64, 1, heads, hd)
        for pos in (0, 1, 7, 40):
            k = rng.standard_normal(elems).astype(np.float32); v = rng.standard_normal(elems).astype(np.float32)
            dk, dv = dev.up(k), dev.up(v)
            dev.call("m40llm_kvcache_append_token_f32_rope_k_at_layout_async", kv_a.h, 0, dk.ptr, dv.ptr, pos, 999, base, 1.0, layout)
            dk2 = dev.up(k)
            dev.call("m40llm_rope_f32_inplace_layout_async", dk2.ptr, 1, heads, hd, pos, base, 1.0, layout)
            dev.call("m40llm_kvcache_reset", kv_b.h)
            dev.call("m40llm_kvcache_append_token_f32", kv_b.h, 0, dk2.ptr, dv.ptr)
            dpos = dev.up(np.array([pos], dtype=np.uint32))
            dev.call("m40llm_kvcache_append_token_f32_rope_k_position_dev_layout_async", kv_c.h, 0, dk.ptr, dv.ptr, dpos.ptr, base, 1.0, layout)
            dev.sync()
            ka, va = kv_a.read_token(0, pos)
            kb, vb = kv_b.read_token(0, 0)
            kc, vc = kv_c.read_token(0, pos)
            assert np.array_equal(ka, kb) and np.array_equal(va, vb)
            assert np.array_equal(ka, kc) and np.array_equal(va, vc)
            assert np.array_equal(va, v.astype(np.float16).view(np.uint16))
            # against the oracle: rotation within tolerance of f16 storage
            Ko = np.zeros((1, 64, heads, hd), dtype=np.uint16); Vo = np.zeros_like(Ko)
            orc.lib().orc_kv_append_f32_rope_k(orc.ptr(Ko), orc.ptr(Vo), 64, heads, hd, 0, pos, orc.ptr(k), orc.ptr(v), base, 1.0, layout)
            # f16 rows of two rotations that differ in the last f32 bit differ by at most one f16 step (2^-10 relative)
            close(ka.view(np.float16).astype(np.float32), Ko[0, pos].reshape(-1).view(np.float16).astype(np.float32))
            assert kv_a.read_raw(5, np.uint32, (1,))[0] == pos + 1      # seq_map = position + 1
        # non-"at" variant stores at the current length and rotates for past_len
        kv_d = m40.KVCache(dev.ctx, 64, 1, heads, hd)
        dev.call("m40llm_kvcache_append_token_f32_rope_k_layout_async", kv_d.h, 0, dk.ptr, dv.ptr, 40, base, 1.0, layout)
        dev.sync()
        kd, _ = kv_d.read_token(0, 0)
        assert np.array_equal(kd, ka)
        dev.call("m40llm_kvcache_append_token_f32_rope_k_at_layout_async", kv_a.h, 0, dk.ptr, dv.ptr, 64, 0, base, 1.0, layout, expect=-5)
        dev.call("m40llm_kvcache_append_token_f32_rope_k_at_layout_async", kv_a.h, 1, dk.ptr, dv.ptr, 0, 0, base, 1.0, layout, expect=-2)


# ------------------------------------------------------------------ GEMM family
@pytest.mark.parametrize("M", [5, 200])
def test_gemm_multi_matrix_equals_separate_calls(dev, M):
    # Q/K/V-shaped and gate/up-shaped groups over shared activations: bit-identical to one GEMM per matrix, for few rows
    # (one GEMM per matrix inside) and many rows (one tiled launch)
    rng = np.random.default_rng(M)
    K, Ns = 256, (384, 64, 136)
    A = rng.standard_normal((M, K)).astype(np.float32)
    Bs = [f16bits(rng.standard_normal((n, K)) * 0.05) for n in Ns]
    dA, dB = dev.up(A), [dev.up(b) for b in Bs]
    for n_mats in (1, 2, 3):
        outs = [dev.zeros(M * n * 4) for n in Ns]
        args = []
        for i in range(3):
            args += [dB[i].ptr, Ns[i], outs[i].ptr] if i < n_mats else [None, 0, None]
        dev.call("m40llm_ext_gemm_f32xf16_gguf_f32_multi_async", dA.ptr, M, K, n_mats, *args, 1)
        dev.sync()
        for i in range(n_mats):
            want = dev.gemm_gguf(A, Bs[i], M, Ns[i], K)
            assert np.array_equal(outs[i].download(np.float32, (M, Ns[i])).view(np.uint32), want.view(np.uint32)), (n_mats, i)
    z = dev.zeros(16)
    dev.call("m40llm_ext_gemm_f32xf16_gguf_f32_multi_async", dA.ptr, M, K, 4, dB[0].ptr, 8, z.ptr, None, 0, None, None, 0, None, 1, expect=-2)
    dev.call("m40llm_ext_gemm_f32xf16_gguf_f32_multi_async", dA.ptr, M, K, 2, dB[0].ptr, 8, z.ptr, None, 8, None, None, 0, None, 1, expect=-1)


@pytest.mark.parametrize("M,N,K", [(33, 16, 32), (100, 200, 2048), (128, 256, 2048), (300, 136, 5632), (257, 2048, 64)])
def test_gemm_many_rows_vs_oracle(dev, orc, M, N, K):
    # the 128 x 128-tile matrix-core GEMM behind m40llm_gemm_f32xf16_gguf_f32 for M > 32 (prefill): ragged tiles in
    # both directions, one and many K steps
    rng = np.random.default_rng(M * 7 + N)
    A = rng.standard_normal((M, K)).astype(np.float32)
    A[1, :8] *= 1e-6                      # tiny activations keep their value through the low part
    B = f16bits(rng.standard_normal((N, K)) * 0.05)
    got = dev.gemm_gguf(A, B, M, N, K)
    want = orc.gemm("f32xf16_gguf", A, B, M, N, K)
    close(got, want)
    # any finite f32 magnitude is carried (the rows are scaled by powers of two before the f16 split) ...
    A[0, ::7] = 1.2e5
    A[2, 5 % K] = -3.0e30
    A[5, :] *= 1e-30
    got = dev.gemm_gguf(A, B, M, N, K)
    want = orc.gemm("f32xf16_gguf", A, B, M, N, K)
    assert np.isfinite(got).all()
    for r in (0, 2, 5):
        close(got[r], want[r], RTOL, RTOL * np.abs(want[r]).max())
    rest = [r for r in range(M) if r not in (0, 2, 5)]
    close(got[rest], want[rest])
    # ... and an infinity or a NaN makes its row non-finite, as in the reference's f32 arithmetic, and no other row
    A[3, 4 % K] = np.inf
    A[4, 9 % K] = np.nan
    bad = dev.gemm_gguf(A, B, M, N, K)
    assert not np.isfinite(bad[3]).any() and np.isnan(bad[4]).all()
    keep = [r for r in range(M) if r not in (3, 4)]
    assert np.array_equal(bad[keep].view(np.uint32), got[keep].view(np.uint32))


@pytest.mark.parametrize("M,N,K", [(2100, 4000, 96), (2100, 4000, 352), (4100, 2056, 2048)])
def test_gemm_wide_tile_vs_float64_oracle_rows_and_narrow_kernel(dev, orc, M, N, K):
    # Grids from 9/16 of a 128 x 256 tile per CU on take the wide-tile kernel (direct global-to-LDS loads, five buffers):
    # fewer K steps than buffers, one turn of its ten-step ring plus a remainder, and many turns; ragged in M and N.
    # Per element within 1e-4 relative + 1e-5 absolute of the float64 product; the first rows also against the oracle's
    # f32 x f16 product (cuda/kernels.cu:5037-5052); and bit for bit what the 128 x 128 kernel gives for the same rows
    # (a call with 1000 rows is too small a grid for the wide tile and too large for a K split: both kernels add a step's
    # high and low products in the same order)
    rng = np.random.default_rng(M + N + K)
    A = rng.standard_normal((M, K)).astype(np.float32)
    A[1, :8] *= 1e-6
    B = f16bits(rng.standard_normal((N, K)) * 0.05)
    got = dev.gemm_gguf(A, B, M, N, K)
    want = A.astype(np.float64) @ B.view(np.float16).astype(np.float64).T
    close(got, want, 1e-4, 1e-5 * np.sqrt(K / 32.0))
    close(got[:24], orc.gemm("f32xf16_gguf", A[:24], B, 24, N, K))
    for r0 in (0, M - 1000):
        narrow = dev.gemm_gguf(np.ascontiguousarray(A[r0:r0 + 1000]), B, 1000, N, K)
        assert np.array_equal(narrow.view(np.uint32), got[r0:r0 + 1000].view(np.uint32)), r0
    assert np.array_equal(dev.gemm_gguf(A, B, M, N, K).view(np.uint32), got.view(np.uint32))      # the same bits on a second call


def test_gemm_wide_tile_multi_matrix_equals_separate_calls(dev):
    # three matrices side by side in one wide-tile launch (8 + 2 + 1 tile columns x 32 tile rows): the same bits as one
    # call per matrix, whichever kernel those calls take
    M, K, Ns = 4096, 256, (2048, 264, 136)
    rng = np.random.default_rng(11)
    A = rng.standard_normal((M, K)).astype(np.float32)
    Bs = [f16bits(rng.standard_normal((n, K)) * 0.05) for n in Ns]
    dA, dB = dev.up(A), [dev.up(b) for b in Bs]
    outs = [dev.zeros(M * n * 4) for n in Ns]
    args = []
    for i in range(3):
        args += [dB[i].ptr, Ns[i], outs[i].ptr]
    dev.call("m40llm_ext_gemm_f32xf16_gguf_f32_multi_async", dA.ptr, M, K, 3, *args, 1)
    dev.sync()
    for i in range(3):
        got = outs[i].download(np.float32, (M, Ns[i]))
        assert np.array_equal(got.view(np.uint32), dev.gemm_gguf(A, Bs[i], M, Ns[i], K).view(np.uint32)), i
        close(got, A.astype(np.float64) @ Bs[i].view(np.float16).astype(np.float64).T, 1e-4, 1e-5 * np.sqrt(K / 32.0))


def test_gemm_known_answers(dev, orc):
    A = f16bits([[1, 2], [3, 4]]); B = f16bits([[5, 6], [7, 8]])
    dA, dB, dC = dev.up(A), dev.up(B), dev.zeros(16)
    dev.call("m40llm_gemm_f16xf16_f32", dA.ptr, dB.ptr, dC.ptr, 2, 2, 2)
    assert np.array_equal(dC.download(np.float32, (2, 2)), [[19, 22], [43, 50]])
    A = f16bits([[1, 2, 3]]); B = f16bits([[4, 5], [6, 7], [8, 9]])
    dA, dB = dev.up(A), dev.up(B)
    dev.call("m40llm_gemm_f16xf16_f32", dA.ptr, dB.ptr, dC.ptr, 1, 2, 3)
    assert np.array_equal(dC.download(np.float32, (1, 2)), [[40, 46]])
    Af = dev.up(np.array([[1, 2, 3]], dtype=np.float32))
    dev.call("m40llm_gemm_f32xf16_f32", Af.ptr, dB.ptr, dC.ptr, 1, 2, 3)
    assert np.array_equal(dC.download(np.float32, (1, 2)), [[40, 46]])
    Bg = dev.up(f16bits(np.array([[4, 5], [6, 7], [8, 9]]).T))
    dev.call("m40llm_gemm_f32xf16_gguf_f32", Af.ptr, Bg.ptr, dC.ptr, 1, 2, 3)
    assert np.array_equal(dC.download(np.float32, (1, 2)), [[40, 46]])
    dC16 = dev.zeros(8)
    dA = dev.up(f16bits([[1, 2], [3, 4]])); dB = dev.up(f16bits([[5, 6], [7, 8]]))
    dev.call("m40llm_gemm_f16_storage_f32_compute", dA.ptr, dB.ptr, dC16.ptr, 2, 2, 2)
    assert np.array_equal(dC16.download(np.uint16, (2, 2)).view(np.float16).astype(np.float32), [[19, 22], [43, 50]])
    assert dev.lib.m40llm_gemm_f32xf16_gguf_f32(None, Af.ptr, Bg.ptr, dC.ptr, 1, 2, 3) == -1
    # tests/gemm_mixed.rs:216-272: GGUF f16 weights materialised as f32 [K][N], then the f32 x f32 product
    a = np.array([[1.0, -2.0, 3.0], [0.5, 4.0, -1.0]], dtype=np.float32)
    b = np.array([0.25, 0.5, 0.75, -1.0, -1.25, 1.5, 2.0, -0.5, 0.125, 3.0, 2.5, -2.0], dtype=np.float32).reshape(4, 3)   # [N][K]
    da, db, dbt, dc = dev.up(a), dev.up(f16bits(b)), dev.zeros(3 * 4 * 4), dev.zeros(2 * 4 * 4)
    dev.call("m40llm_materialize_gguf_f16_to_f32_colmajor_nt", db.ptr, dbt.ptr, 4, 3)
    assert np.array_equal(dbt.download(np.float32, (3, 4)), b.T)
    dev.call("m40llm_gemm_f32xf32_f32", da.ptr, dbt.ptr, dc.ptr, 2, 4, 3)
    assert np.array_equal(dc.download(np.float32, (2, 4)), a @ b.T)      # small dyadic values: exact
    dev.call("m40llm_gemm_f32xf32_f32", da.ptr, dbt.ptr, dc.ptr, 0, 4, 3, expect=-2)


@pytest.mark.parametrize("M,N,K", [
    (1, 2048, 2048), (1, 256, 2048), (1, 5632, 2048), (1, 2048, 5632), (1, 32000, 2048),   # TinyLlama shapes
    (1, 11008, 2048), (1, 2048, 11008),                                                        # Qwen2.5-3B shapes
    (2, 2048, 2048), (4, 256, 2048), (8, 2048, 2048), (7, 333, 1024), (8, 8192, 256), (6, 4100, 2048),   # row-batched vector-ALU kernel
    (8, 11008, 2048), (8, 2048, 11008), (3, 9000, 2048), (8, 512, 4096),                       # batched (MFMA, stacked)
    (16, 2048, 2048), (9, 4096, 4096), (16, 300, 14336),                                       # MFMA, two fragment sets
    (20, 520, 1024),                                                                           # more than one row tile
    (1, 37, 300), (3, 37, 300), (5, 7, 8), (1, 50, 2056),                                      # odd shapes: generic / tails
])
def test_gemm_gguf_vs_oracle(dev, orc, M, N, K):
    rng = np.random.default_rng(M * 1000003 + N * 101 + K)
    A = rng.standard_normal((M, K)).astype(np.float32)
    if M > 1:
        A[1] *= 1e-3          # rows of very different magnitude (per-row scaling of the hi/lo split)
    if M > 2:
        A[2] *= 3e4
    B = f16bits(rng.standard_normal((N, K)) * 0.02)
    got = dev.gemm_gguf(A, B, M, N, K)
    want = orc.gemm("f32xf16_gguf", A, B, M, N, K)
    scale = np.abs(want).max(axis=1, keepdims=True)
    # relative 1e-3 / absolute 1e-4 on rows normalised to unit scale
    close(got / scale, want / scale)
    f64 = A.astype(np.float64) @ B.view(np.float16).astype(np.float64).T
    close(got / scale, f64 / scale, 1e-4, 1e-5)


def test_gemm_batched_rows_match_single_row(dev, orc):
    """Each row of the batched (MFMA) GEMM is the same dot product as the M=1 GEMV within tolerance, and does
    not depend on which other rows share the batch."""
    rng = np.random.default_rng(5)
    N, K = 2048, 2048
    B = f16bits(rng.standard_normal((N, K)) * 0.02)
    A = rng.standard_normal((8, K)).astype(np.float32)
    full = dev.gemm_gguf(A, B, 8, N, K)
    A2 = A.copy(); A2[[0, 2, 4]] = rng.standard_normal((3, K)).astype(np.float32) * 100
    part = dev.gemm_gguf(A2, B, 8, N, K)
    assert np.array_equal(full[[1, 3, 5, 6, 7]], part[[1, 3, 5, 6, 7]])
    single = dev.gemm_gguf(A[3:4], B, 1, N, K)
    close(full[3:4], single, 1e-4, 1e-5)


def test_gemm_async_extension_matches_blocking(dev, orc):
    rng = np.random.default_rng(6)
    M, N, K = 1, 4096, 2048
    A = rng.standard_normal((M, K)).astype(np.float32); B = f16bits(rng.standard_normal((N, K)) * 0.02)
    dA, dB, dC = dev.up(A), dev.up(B), dev.zeros(M * N * 4)
    dev.call("m40llm_ext_gemm_f32xf16_gguf_f32_async", dA.ptr, dB.ptr, dC.ptr, M, N, K, 1)
    dev.sync()
    assert np.array_equal(dC.download(np.float32, (M, N)), dev.gemm_gguf(A, B, M, N, K))
    dev.call("m40llm_ext_gemm_f32xf16_gguf_f32_async", dA.ptr, dB.ptr, dC.ptr, M, N, K, 2, expect=-4)


def test_gemm_rowmajor_vs_oracle(dev, orc):
    rng = np.random.default_rng(7)
    M, N, K = 5, 300, 129
    A = rng.standard_normal((M, K)).astype(np.float32); B = f16bits(rng.standard_normal((K, N)) * 0.1)
    dA, dB, dC = dev.up(A), dev.up(B), dev.zeros(M * N * 4)
    dev.call("m40llm_gemm_f32xf16_f32", dA.ptr, dB.ptr, dC.ptr, M, N, K)
    close(dC.download(np.float32, (M, N)), orc.gemm("f32xf16_rowmajor", A, B, M, N, K), 1e-4, 1e-5)
    A16 = f16bits(A); dA16 = dev.up(A16)
    dev.call("m40llm_gemm_f16xf16_f32", dA16.ptr, dB.ptr, dC.ptr, M, N, K)
    close(dC.download(np.float32, (M, N)), orc.gemm("f16xf16_rowmajor", A16, B, M, N, K), 1e-4, 1e-5)


@pytest.mark.parametrize("M", [1, 2, 4, 16])
def test_q80_gemm_and_ffn_vs_oracle(dev, orc, M):
    rng = np.random.default_rng(11 + M)
    d_model, ffn = 256, 512
    def qmat(n, k):
        d = rng.uniform(0.001, 0.01, size=(n, k // 32)).astype(np.float16)
        qs = rng.integers(-127, 128, size=(n, k // 32, 32)).astype(np.int8)
        return np.ascontiguousarray(np.stack([_q80_pack(d[i], qs[i]) for i in range(n)]))
    wg, wu, wd = qmat(ffn, d_model), qmat(ffn, d_model), qmat(d_model, ffn)
    x = rng.standard_normal((M, d_model)).astype(np.float32)
    dx, dwg, dC = dev.up(x), dev.up(wg), dev.zeros(M * ffn * 4)
    dev.call("m40llm_ext_gemm_f32xq80_gguf_f32", dx.ptr, dwg.ptr, dC.ptr, M, ffn, d_model)
    want = orc.gemm("f32xq80_gguf", x, wg, M, ffn, d_model)
    close(dC.download(np.float32, (M, ffn)), want, 1e-3, 1e-4 * np.abs(want).max())
    dwu, dwd = dev.up(wu), dev.up(wd)
    scratch, out = dev.zeros(2 * M * ffn * 4), dev.zeros(M * d_model * 4)
    dev.call("m40llm_ext_ffn_swiglu_q80_f32_async", dx.ptr, dwg.ptr, dwu.ptr, dwd.ptr, scratch.ptr, out.ptr, M, d_model, ffn)
    dev.sync()
    want = orc.ffn_swiglu_q80(x, wg, wu, wd, M, d_model, ffn)
    close(out.download(np.float32, (M, d_model)), want, 1e-3, 1e-4 * max(np.abs(want).max(), 1.0))


@pytest.fixture(scope="module")
def q80_ffn_full_size():
    """q8_0 gate / up / down of BASELINE config 4 (hidden 4096, FFN 14336): int8 uniform in [-127, 127], f16 scales
    U(0.001, 0.01), built once for the rows-per-call cases below."""
    rng = np.random.default_rng(404)
    def qmat(n, k):
        blob = np.empty((n, k // 32, 34), dtype=np.uint8)
        blob[:, :, :2] = rng.uniform(0.001, 0.01, size=(n, k // 32)).astype(np.float16).view(np.uint8).reshape(n, k // 32, 2)
        blob[:, :, 2:] = rng.integers(-127, 128, size=(n, k // 32, 32)).astype(np.int8).view(np.uint8)
        return blob
    return qmat(14336, 4096), qmat(14336, 4096), qmat(4096, 14336)


@pytest.mark.parametrize("M", [1, 2, 4, 7, 16])
def test_q80_ffn_full_size_vs_oracle(dev, orc, q80_ffn_full_size, M):
    """The fused q8_0 FFN at the full BASELINE config 4 size, batch sizes 1, 2, 4, 7 and 16, against the oracle's sequential
    f32 sums: 1e-3 relative / 1e-4 absolute on outputs scaled to a unit row maximum (7 and 16 rows: the two paddings of
    the three-plane int8 form)."""
    wg, wu, wd = q80_ffn_full_size
    d_model, ffn = 4096, 14336
    x = np.random.default_rng(40 + M).standard_normal((M, d_model)).astype(np.float32)
    dx, dwg, dwu, dwd = dev.up(x), dev.up(wg), dev.up(wu), dev.up(wd)
    scratch, out = dev.zeros(2 * M * ffn * 4), dev.zeros(M * d_model * 4)
    dev.call("m40llm_ext_ffn_swiglu_q80_f32_async", dx.ptr, dwg.ptr, dwu.ptr, dwd.ptr, scratch.ptr, out.ptr, M, d_model, ffn)
    dev.sync()
    orc.set_threads(8)
    want = orc.ffn_swiglu_q80(x, wg, wu, wd, M, d_model, ffn)
    scale = np.abs(want).max(axis=1, keepdims=True)
    got = out.download(np.float32, (M, d_model))
    close(got / scale, want / scale, 1e-3, 1e-4)
    # twice the same call: the same bits (the down projection adds two halves of K into a cleared result: 0 + a + b)
    dev.call("m40llm_ext_ffn_swiglu_q80_f32_async", dx.ptr, dwg.ptr, dwu.ptr, dwd.ptr, scratch.ptr, out.ptr, M, d_model, ffn)
    dev.sync()
    assert np.array_equal(out.download(np.float32, (M, d_model)), got)
    if M in (4, 16):
        # result written over the input rows
        dev.call("m40llm_ext_ffn_swiglu_q80_f32_async", dx.ptr, dwg.ptr, dwu.ptr, dwd.ptr, scratch.ptr, dx.ptr, M, d_model, ffn)
        dev.sync()
        close(dx.download(np.float32, (M, d_model)) / scale, want / scale, 1e-3, 1e-4)


@pytest.mark.parametrize("M,d_model", [(3, 1024), (4, 768), (2, 2048)])
def test_q80_ffn_wide_hidden_short_k_vs_oracle(dev, orc, M, d_model):
    """A wide FFN (12288 hidden columns: the launch shape whose workgroups pack the activation rows themselves) over a
    short K, where some of the packing passes have no block to pack; 768 = 3 steps, 1024 = 4, 2048 = 8."""
    rng = np.random.default_rng(500 + M)
    ffn = 12288
    def qmat(n, k):
        blob = np.empty((n, k // 32, 34), dtype=np.uint8)
        blob[:, :, :2] = rng.uniform(0.001, 0.01, size=(n, k // 32)).astype(np.float16).view(np.uint8).reshape(n, k // 32, 2)
        blob[:, :, 2:] = rng.integers(-127, 128, size=(n, k // 32, 32)).astype(np.int8).view(np.uint8)
        return blob
    wg, wu, wd = qmat(ffn, d_model), qmat(ffn, d_model), qmat(d_model, ffn)
    x = rng.standard_normal((M, d_model)).astype(np.float32)
    x[M - 1] *= 1e-3
    dx, dwg, dwu, dwd = dev.up(x), dev.up(wg), dev.up(wu), dev.up(wd)
    scratch, out = dev.zeros(2 * M * ffn * 4), dev.zeros(M * d_model * 4)
    dev.call("m40llm_ext_ffn_swiglu_q80_f32_async", dx.ptr, dwg.ptr, dwu.ptr, dwd.ptr, scratch.ptr, out.ptr, M, d_model, ffn)
    dev.sync()
    orc.set_threads(8)
    want = orc.ffn_swiglu_q80(x, wg, wu, wd, M, d_model, ffn)
    scale = np.abs(want).max(axis=1, keepdims=True)
    close(out.download(np.float32, (M, d_model)) / scale, want / scale, 1e-3, 1e-4)


@pytest.mark.parametrize("M,N,K", [(1, 300, 512), (3, 1000, 768), (8, 4096, 2048), (9, 520, 1280), (16, 2048, 4096),
                                   (20, 333, 256), (2, 64, 96), (1, 1000, 4096), (2, 777, 8192), (1, 513, 14336),
                                   (2, 260, 11008), (1, 40, 16384), (2, 3, 64), (8, 6200, 512), (12, 24600, 256),
                                   (5, 8192, 1024), (4, 12300, 512), (6, 3100, 8192), (3, 4096, 8192)])
def test_q80_gemm_shapes_vs_oracle(dev, orc, M, N, K):
    """MFMA path (3 rows and more, K % 256 == 0; column tails, split K, more than 16 rows; 5 rows and more with 6144
    columns and more: two column tiles per wave, split K and, from ~24 500 columns, whole K; ~3100 to 16 000 columns with
    K of 8192 and more: tile pairs x two halves of K added into a cleared result), the register-resident
    GEMV of one and two rows (K % 64 == 0, one, two and four K-parts per column) and the simple path (K = 96)."""
    rng = np.random.default_rng(M * 7919 + N + K)
    d = rng.uniform(0.001, 0.01, size=(N, K // 32)).astype(np.float16)
    qs = rng.integers(-127, 128, size=(N, K // 32, 32)).astype(np.int8)
    qs[0, 0, :] = -127; qs[N - 1, -1, :] = 127; qs[N // 2, 0, ::2] = 0          # extremes of the int8 -> f16 step
    W = np.ascontiguousarray(np.stack([_q80_pack(d[i], qs[i]) for i in range(N)]))
    A = rng.standard_normal((M, K)).astype(np.float32)
    if M > 1:
        A[1] *= 1e-3
    if M > 2:
        A[2] *= 3e4
    dA, dW, dC = dev.up(A), dev.up(W), dev.zeros(M * N * 4)
    dev.call("m40llm_ext_gemm_f32xq80_gguf_f32", dA.ptr, dW.ptr, dC.ptr, M, N, K)
    got = dC.download(np.float32, (M, N))
    want = orc.gemm("f32xq80_gguf", A, W, M, N, K)
    scale = np.abs(want).max(axis=1, keepdims=True)
    close(got / scale, want / scale)
    f64 = A.astype(np.float64) @ (d.astype(np.float64)[:, :, None] * qs.astype(np.float64)).reshape(N, K).T
    close(got / scale, f64 / scale, 1e-4, 1e-5)


def test_q80_gemv_random_shapes_vs_float64(dev):
    """One and two rows over seeded random shapes: K = 64..16384 in steps of 64 (one to eight K parts per column,
    partly filled parts, lanes without a block), N from 1 up (fewer columns than teams, column tails).  The matrix
    buffer is exactly N * K/32 * 34 bytes, so a read outside it would land outside the allocation's payload."""
    rng = np.random.default_rng(2024)
    shapes = [(1, 1, 64), (2, 1, 128), (1, 17, 16384), (2, 5, 16320), (1, 3, 4160), (2, 2, 2112)]
    for _ in range(18):
        shapes.append((int(rng.integers(1, 3)), int(rng.integers(1, 400)), 64 * int(rng.integers(1, 130))))
    for M, N, K in shapes:
        d = rng.uniform(0.001, 0.01, size=(N, K // 32)).astype(np.float16)
        qs = rng.integers(-127, 128, size=(N, K // 32, 32)).astype(np.int8)
        W = np.ascontiguousarray(np.stack([_q80_pack(d[i], qs[i]) for i in range(N)]))
        A = rng.standard_normal((M, K)).astype(np.float32)
        dA, dW, dC = dev.up(A), dev.up(W), dev.zeros(M * N * 4)
        dev.call("m40llm_ext_gemm_f32xq80_gguf_f32", dA.ptr, dW.ptr, dC.ptr, M, N, K)
        got = dC.download(np.float32, (M, N))
        f64 = A.astype(np.float64) @ (d.astype(np.float64)[:, :, None] * qs.astype(np.float64)).reshape(N, K).T
        scale = np.abs(f64).max(axis=1, keepdims=True)
        close(got / scale, f64 / scale, 1e-4, 1e-5)
        dA.free(); dW.free(); dC.free()


def test_q80_int8_forms_seeded_shapes_vs_float64(dev):
    """The int8 matrix-instruction forms over seeded shapes: 2 to 16 rows (stacked and three-plane form), column counts on
    both sides of every launch-shape switch (whole K / split K / two tiles per wave / two halves of K added into a cleared
    result) with ragged tails, K from one step (256) to 40; against float64 of the same operands."""
    rng = np.random.default_rng(90210)
    shapes = [(3, 17, 256), (16, 1, 512), (5, 6143, 256), (5, 6145, 512), (4, 12287, 256), (4, 12289, 512), (9, 3071, 8192),
              (9, 3073, 8192), (2, 3073, 10240), (16, 16385, 256), (7, 8209, 1024), (13, 24577, 256), (4, 8193, 2048)]
    for _ in range(10):
        shapes.append((int(rng.integers(3, 17)), int(rng.integers(1, 9000)), 256 * int(rng.integers(1, 9))))
    for M, N, K in shapes:
        d = rng.uniform(0.001, 0.01, size=(N, K // 32)).astype(np.float16)
        qs = rng.integers(-127, 128, size=(N, K // 32, 32)).astype(np.int8)
        W = np.empty((N, K // 32, 34), dtype=np.uint8)
        W[:, :, :2] = d.view(np.uint8).reshape(N, K // 32, 2)
        W[:, :, 2:] = qs.view(np.uint8)
        A = rng.standard_normal((M, K)).astype(np.float32)
        A[M - 1] *= 1e-4
        A[0, ::7] *= 50.0
        dA, dW, dC = dev.up(A), dev.up(W), dev.up(np.full((M, N), 3.0, dtype=np.float32))
        dev.call("m40llm_ext_gemm_f32xq80_gguf_f32", dA.ptr, dW.ptr, dC.ptr, M, N, K)
        got = dC.download(np.float32, (M, N))
        f64 = A.astype(np.float64) @ (d.astype(np.float64)[:, :, None] * qs.astype(np.float64)).reshape(N, K).T
        scale = np.abs(f64).max(axis=1, keepdims=True)
        close(got / scale, f64 / scale, 1e-4, 1e-5)
        dA.free(); dW.free(); dC.free()


def _q80_const_matrix(n, k, scale, pattern):
    """q8_0 matrix whose column c holds the single quant pattern[c % len(pattern)] in every block (scale as f16)."""
    W = np.empty((n, k // 32, 34), dtype=np.uint8)
    W[:, :, :2] = np.full((n, k // 32), scale, dtype=np.float16).view(np.uint8).reshape(n, k // 32, 2)
    q = np.array([pattern[c % len(pattern)] for c in range(n)], dtype=np.int8)
    W[:, :, 2:] = np.broadcast_to(q.view(np.uint8)[:, None, None], (n, k // 32, 32))
    dense = np.float64(np.float16(scale)) * np.broadcast_to(q.astype(np.float64)[:, None], (n, k))
    return W, dense


@pytest.mark.parametrize("M", [3, 5, 16])
def test_q80_int8_like_signed_blocks_vs_float64(dev, M):
    """Blocks whose activations all have one sign and one size against columns of one large quant (127 or -128): the
    integer block sum of the three-digit form reaches 2^32 there (x = 0.9, 0.6, -1, 0.99 are the cases that wrapped a
    32-bit recombination).  GEMM and fused FFN, stacked (3 rows) and three-plane form (5, 16 rows), against float64."""
    K, N = 512, 96
    W, dense = _q80_const_matrix(N, K, 0.0078125, [127, -128, 80, -127])
    vals = [0.9, 0.6, -1.0, 0.99, 0.5, -0.9, 1.0, 0.75]
    A = np.empty((M, K), dtype=np.float32)
    for m in range(M):
        A[m] = vals[m % len(vals)]
    A[M - 1, 32:64] = -0.9                                  # one block of the other sign
    dA, dW, dC = dev.up(A), dev.up(W), dev.zeros(M * N * 4)
    dev.call("m40llm_ext_gemm_f32xq80_gguf_f32", dA.ptr, dW.ptr, dC.ptr, M, N, K)
    got = dC.download(np.float32, (M, N))
    f64 = A.astype(np.float64) @ dense.T
    scale = np.abs(f64).max(axis=1, keepdims=True)
    close(got / scale, f64 / scale, 1e-5, 1e-6)
    # fused FFN: gate columns of both signs, up and down of one sign each; long K for the two-halves down projection too
    for d_model, ffn in ((512, 1024), (3072, 8192)):
        wg, g64 = _q80_const_matrix(ffn, d_model, 0.001, [127, -128, 64, -3])
        wu, u64 = _q80_const_matrix(ffn, d_model, 0.002, [127, 127, -128, 90])
        wd, d64 = _q80_const_matrix(d_model, ffn, 0.001, [127, -128])
        x = np.ascontiguousarray(np.tile(A[:, :256], (1, d_model // 256))) * np.float32(0.125)
        dx, dwg, dwu, dwd = dev.up(x), dev.up(wg), dev.up(wu), dev.up(wd)
        scratch, out = dev.zeros(2 * M * ffn * 4), dev.zeros(M * d_model * 4)
        dev.call("m40llm_ext_ffn_swiglu_q80_f32_async", dx.ptr, dwg.ptr, dwu.ptr, dwd.ptr, scratch.ptr, out.ptr, M, d_model, ffn)
        dev.sync()
        g = x.astype(np.float64) @ g64.T
        h = g / (1.0 + np.exp(-g)) * (x.astype(np.float64) @ u64.T)
        want = h @ d64.T
        scale = np.abs(want).max(axis=1, keepdims=True)
        close(out.download(np.float32, (M, d_model)) / scale, want / scale, 1e-4, 1e-5)
        for b in (dx, dwg, dwu, dwd, scratch, out):
            b.free()


@pytest.mark.parametrize("M", [2, 4, 5, 16])
def test_q80_non_finite_activations_stay_non_finite(dev, M):
    """A NaN or an infinity in an activation row reaches every output of that row as a non-finite value on every q8_0
    path (register GEMV at 2 rows, stacked int8 form at 4, three-plane form at 5 and 16), as the f32 product of the
    reference does (kernels.cu:5037-5052); the other rows are unaffected."""
    rng = np.random.default_rng(77 + M)
    N, K = 160, 512
    d = rng.uniform(0.001, 0.01, size=(N, K // 32)).astype(np.float16)
    qs = rng.integers(-127, 128, size=(N, K // 32, 32)).astype(np.int8)
    qs[qs == 0] = 1
    W = np.empty((N, K // 32, 34), dtype=np.uint8)
    W[:, :, :2] = d.view(np.uint8).reshape(N, K // 32, 2)
    W[:, :, 2:] = qs.view(np.uint8)
    A = rng.standard_normal((M, K)).astype(np.float32)
    clean = A.copy()
    A[0, 37] = np.nan
    A[1, 300] = np.inf
    dA, dW, dC = dev.up(A), dev.up(W), dev.zeros(M * N * 4)
    dev.call("m40llm_ext_gemm_f32xq80_gguf_f32", dA.ptr, dW.ptr, dC.ptr, M, N, K)
    got = dC.download(np.float32, (M, N))
    assert not np.isfinite(got[0]).any() and not np.isfinite(got[1]).any()
    assert np.isnan(got[0]).all()
    if M > 2:
        f64 = clean.astype(np.float64) @ (d.astype(np.float64)[:, :, None] * qs.astype(np.float64)).reshape(N, K).T
        scale = np.abs(f64[2:]).max(axis=1, keepdims=True)
        close(got[2:] / scale, f64[2:] / scale, 1e-4, 1e-5)


# ------------------------------------------------------------------ dense attention
def _attention_case(dev, orc, qh, kvh, hd, L, k, v, q, max_seq=None, seq=0, batch=1):
    max_seq = max_seq or L
    kv = m40.KVCache(dev.ctx, max_seq, batch, kvh, hd)
    K16 = f16bits(k).reshape(L, kvh, hd); V16 = f16bits(v).reshape(L, kvh, hd)
    dev.fill_dense(kv, seq, K16, V16)
    got = dev.attention(kv, seq, q, qh, L)
    Kc = np.zeros((batch, max_seq, kvh, hd), dtype=np.uint16); Vc = np.zeros_like(Kc)
    Kc[seq, :L] = K16; Vc[seq, :L] = V16
    want = orc.attention(Kc, Vc, max_seq, kvh, hd, seq, q, qh, L)
    return got, want, kv


def test_attention_mha_grid_fixture(dev, orc):
    # grid + closed-form data of tests/attention_parity_cpu_grid.rs:74-118, via the MHA entry point
    for heads in (1, 2, 3, 4):
        for hd in (1, 5, 7, 8, 16, 31, 32, 63, 64):
            dim = heads * hd
            for L in (1, 2, 3, 4, 7, 8, 16):
                t = np.arange(L)[:, None]; i = np.arange(dim)[None, :]
                k = ((t * dim + i).astype(np.float32) * np.float32(0.01) - 1)
                v = ((t * dim + (dim - 1 - i)).astype(np.float32) * np.float32(0.02) - 2)
                q = (np.arange(dim, dtype=np.float32) * np.float32(0.003) - np.float32(0.5))
                kv = m40.KVCache(dev.ctx, 16, 1, heads, hd)
                for tt in range(L):
                    dk, dv = dev.up(k[tt].astype(np.float32)), dev.up(v[tt].astype(np.float32))
                    dev.call("m40llm_kvcache_append_token_f32_async", kv.h, 0, dk.ptr, dv.ptr)
                dq, out = dev.up(q), dev.zeros(dim * 4)
                dev.call("m40llm_attention_last_token_f32", kv.h, 0, dq.ptr, L, out.ptr)
                Kc = np.zeros((1, 16, heads, hd), dtype=np.uint16); Vc = np.zeros_like(Kc)
                Kc[0, :L] = f16bits(k).reshape(L, heads, hd); Vc[0, :L] = f16bits(v).reshape(L, heads, hd)
                want = orc.attention(Kc, Vc, 16, heads, hd, 0, q, heads, L)
                close(out.download(np.float32, (dim,)), want, 1e-3, 1e-4)   # tests/attention_last_token.rs:203
                kv.destroy()


@pytest.mark.parametrize("L", [128, 512])
def test_attention_gqa_config1_reference_fixture(dev, orc, L):
    qh, kvh, hd = 32, 4, 64           # tests/attention_parity_cuda_grid.rs:1737-1772
    kv_dim = kvh * hd
    t = np.arange(L)[:, None]; i = np.arange(kv_dim)[None, :]
    k = ((t * kv_dim + i).astype(np.float32) * np.float32(0.0003) - np.float32(0.25))
    v = ((t * kv_dim + (kv_dim - 1 - i)).astype(np.float32) * np.float32(0.0002) - np.float32(0.1))
    q = (np.arange(qh * hd, dtype=np.float32) * np.float32(0.0004) - np.float32(0.2))
    got, want, _ = _attention_case(dev, orc, qh, kvh, hd, L, k, v, q)
    close(got, want)


@pytest.mark.parametrize("qh,kvh,hd,L", [
    (32, 4, 64, 512),        # BASELINE config 1 (seed 0, N(0,1))
    (32, 4, 64, 1), (32, 4, 64, 33), (32, 4, 64, 160),
    (16, 2, 128, 2176), (16, 2, 128, 4096),
    (32, 8, 128, 9000),      # beyond the reference's 8192 fast-path cap
    (6, 2, 64, 100), (3, 3, 128, 70), (12, 1, 64, 257), (5, 1, 128, 31),   # uneven groups
])
def test_attention_random_vs_oracle(dev, orc, qh, kvh, hd, L):
    rng = np.random.default_rng(0)
    q = rng.standard_normal(qh * hd).astype(np.float32)
    k = rng.standard_normal((L, kvh * hd)).astype(np.float32)
    v = rng.standard_normal((L, kvh * hd)).astype(np.float32)
    got, want, kv = _attention_case(dev, orc, qh, kvh, hd, L, k, v, q, max_seq=L + 3, seq=1, batch=2)
    close(got, want)
    if L == 1:
        vf = f16bits(v).view(np.float16).astype(np.float32).reshape(kvh, hd)
        assert np.array_equal(got.reshape(qh, hd), np.repeat(vf, qh // kvh, axis=0))
    # error codes
    dq, out = dev.up(q), dev.zeros(qh * hd * 4)
    dev.call("m40llm_attention_last_token_f32_gqa_async", kv.h, 2, dq.ptr, qh, L, out.ptr, expect=-2)
    dev.call("m40llm_attention_last_token_f32_gqa_async", kv.h, 0, dq.ptr, qh, 0, out.ptr, expect=-3)
    dev.call("m40llm_attention_last_token_f32_gqa_async", kv.h, 0, dq.ptr, qh, L + 4, out.ptr, expect=-3)
    dev.call("m40llm_attention_last_token_f32_gqa_async", kv.h, 0, dq.ptr, qh + 1 if kvh > 1 else 0, L, out.ptr, expect=-6)
    # device-side length and recent-window forms agree with the plain call
    dlen = dev.up(np.array([L], dtype=np.uint32))
    dev.call("m40llm_attention_last_token_f32_gqa_seq_len_dev_async", kv.h, 1, dq.ptr, qh, dlen.ptr, out.ptr)
    dev.sync()
    close(out.download(np.float32, (qh * hd,)), want)
    W = max(1, L // 3)
    dev.call("m40llm_attention_last_token_f32_gqa_dense_recent_async", kv.h, 1, dq.ptr, qh, L, W, out.ptr)
    dev.sync()
    Kc = np.zeros((1, W, kvh, hd), dtype=np.uint16); Vc = np.zeros_like(Kc)
    Kc[0] = f16bits(k).reshape(L, kvh, hd)[L - W:]; Vc[0] = f16bits(v).reshape(L, kvh, hd)[L - W:]
    close(out.download(np.float32, (qh * hd,)), orc.attention(Kc, Vc, W, kvh, hd, 0, q, qh, W))


def test_attention_batched_varlen_reference_fixture(dev, orc):
    # tests/attention_batched_varlen.rs:36-69: qh 4, kvh 2, hd 64, lens [1,3,5], ids [0,1,2]
    qh, kvh, hd, maxL = 4, 2, 64, 8
    kv = m40.KVCache(dev.ctx, maxL, 3, kvh, hd)
    Kc = np.zeros((3, maxL, kvh, hd), dtype=np.uint16); Vc = np.zeros_like(Kc)
    lens, ids = [1, 3, 5], [0, 1, 2]
    for s, L in zip(ids, lens):
        t = np.arange(L)[:, None]; i = np.arange(kvh * hd)[None, :]
        k = ((s * 7 + t * 3 + i) % 17).astype(np.float32) * np.float32(0.05) - np.float32(0.4)
        v = ((s * 5 + t * 11 + i) % 13).astype(np.float32) * np.float32(0.07) - np.float32(0.3)
        Kc[s, :L] = f16bits(k).reshape(L, kvh, hd); Vc[s, :L] = f16bits(v).reshape(L, kvh, hd)
        dev.fill_dense(kv, s, Kc[s, :L], Vc[s, :L])
    q = ((np.arange(3 * qh * hd) % 19).astype(np.float32) * np.float32(0.03) - np.float32(0.25)).reshape(3, qh * hd)
    dq, out = dev.up(q), dev.zeros(q.nbytes)
    dids, dlens = dev.up(np.array(ids, dtype=np.uint32)), dev.up(np.array(lens, dtype=np.uint32))
    dev.call("m40llm_attention_last_token_f32_gqa_batched", kv.h, dids.ptr, dlens.ptr, 3, dq.ptr, qh, out.ptr)
    got = out.download(np.float32, q.shape)
    close(got, orc.attention_batched(Kc, Vc, maxL, kvh, hd, ids, lens, q, qh), 1e-4, 1e-5)   # reference: 1e-4
    for b in range(3):      # batched == individual calls
        close(got[b], dev.attention(kv, ids[b], q[b], qh, lens[b]), 1e-4, 1e-5)
    # validation codes
    dev.call("m40llm_attention_last_token_f32_gqa_batched_async", kv.h, dids.ptr, dlens.ptr, 0, dq.ptr, qh, out.ptr, expect=-2)
    dev.call("m40llm_attention_last_token_f32_gqa_batched_async", kv.h, dids.ptr, dlens.ptr, 3, dq.ptr, 3, out.ptr, expect=-3)
    bad = dev.up(np.array([1, 0, 5], dtype=np.uint32))
    dev.call("m40llm_attention_last_token_f32_gqa_batched_async", kv.h, dids.ptr, bad.ptr, 3, dq.ptr, qh, out.ptr, expect=-8)
    bad = dev.up(np.array([0, 1, 3], dtype=np.uint32))
    dev.call("m40llm_attention_last_token_f32_gqa_batched_async", kv.h, bad.ptr, dlens.ptr, 3, dq.ptr, qh, out.ptr, expect=-8)


def test_attention_batched_head128_qwen_shape(dev, orc):
    # BASELINE config 3 attention shape: 16 q / 2 kv heads, hd 128, 8 sequences, lengths U[256, 4096]
    rng = np.random.default_rng(0)
    qh, kvh, hd, B, maxL = 16, 2, 128, 8, 4160
    lens = rng.integers(256, 4097, size=B).astype(np.uint32)
    ids = rng.permutation(B).astype(np.uint32)
    kv = m40.KVCache(dev.ctx, maxL, B, kvh, hd)
    Kc = np.zeros((B, maxL, kvh, hd), dtype=np.uint16); Vc = np.zeros_like(Kc)
    for b in range(B):
        L = int(lens[b]); s = int(ids[b])
        Kc[s, :L] = f16bits(rng.standard_normal((L, kvh, hd))); Vc[s, :L] = f16bits(rng.standard_normal((L, kvh, hd)))
        dev.fill_dense(kv, s, Kc[s, :L], Vc[s, :L])
    q = rng.standard_normal((B, qh * hd)).astype(np.float32)
    dq, out = dev.up(q), dev.zeros(q.nbytes)
    dids, dlens = dev.up(ids), dev.up(lens)
    dev.call("m40llm_attention_last_token_f32_gqa_batched_async", kv.h, dids.ptr, dlens.ptr, B, dq.ptr, qh, out.ptr)
    dev.sync()
    orc.set_threads(8)
    close(out.download(np.float32, q.shape), orc.attention_batched(Kc, Vc, maxL, kvh, hd, ids, lens, q, qh))


def test_attention_device_lengths_and_skipped_rows(dev, orc):
    """The entry points that read lengths (and ids) on the device: rows inside the bound equal the oracle; a row whose
    length exceeds max_len_hint, a zero-length row and a row with an id outside the cache are skipped (their output rows
    keep what was there), for the chunked (hint > 512) and the single-chunk launch shapes."""
    rng = np.random.default_rng(21)
    qh, kvh, hd, S, maxL = 8, 2, 128, 6, 1536
    kv = m40.KVCache(dev.ctx, maxL, S, kvh, hd)
    Kc = f16bits(rng.standard_normal((S, maxL, kvh, hd))); Vc = f16bits(rng.standard_normal((S, maxL, kvh, hd)))
    for s_ in range(S):
        dev.fill_dense(kv, s_, Kc[s_], Vc[s_])
    for hint, lens in ((1024, [300, 700, 1200, 0, 1024, 50]), (400, [300, 399, 401, 17, 400, 1])):
        lens = np.asarray(lens, dtype=np.uint32)
        ids = np.asarray([3, 0, 1, 2, 5, 9], dtype=np.uint32)          # id 9 does not exist
        B = len(lens)
        q = rng.standard_normal((B, qh * hd)).astype(np.float32)
        sentinel = np.full(q.shape, 7.25, dtype=np.float32)
        dq, out, dids, dlens = dev.up(q), dev.up(sentinel), dev.up(ids), dev.up(lens)
        dev.call("m40llm_ext_attention_last_token_f32_gqa_batched_lens_dev_async", kv.h, dids.ptr, dlens.ptr, 0, B, hint,
                 dq.ptr, qh, out.ptr)
        dev.sync()
        got = out.download(np.float32, q.shape)
        live = [b for b in range(B) if 0 < lens[b] <= hint and ids[b] < S]
        assert 3 <= len(live) < B
        want = orc.attention_batched(Kc, Vc, maxL, kvh, hd, ids[live], lens[live], q[live], qh)
        close(got[live], want)
        for b in range(B):
            if b not in live:
                assert np.array_equal(got[b], sentinel[b]), b
    # single sequence, length = *position_dev + 1
    q = rng.standard_normal((1, qh * hd)).astype(np.float32)
    for pos, hint, skipped in ((699, 1024, False), (699, 700, False), (700, 700, True), (99, 128, False), (128, 128, True)):
        sentinel = np.full(q.shape, -3.5, dtype=np.float32)
        dq, out, dpos = dev.up(q), dev.up(sentinel), dev.up(np.asarray([pos], dtype=np.uint32))
        dev.call("m40llm_ext_attention_last_token_f32_gqa_position_dev_async", kv.h, 4, dq.ptr, qh, dpos.ptr, hint, out.ptr)
        dev.sync()
        got = out.download(np.float32, q.shape)
        if skipped:
            assert np.array_equal(got, sentinel)
        else:
            close(got, orc.attention_batched(Kc, Vc, maxL, kvh, hd, np.asarray([4], np.uint32), np.asarray([pos + 1], np.uint32), q, qh))
    dev.call("m40llm_ext_attention_last_token_f32_gqa_position_dev_async", kv.h, 4, dq.ptr, qh, dpos.ptr, maxL + 1, out.ptr, expect=-3)


def test_argmax_extension(dev, orc):
    rng = np.random.default_rng(9)
    rows, n = 8, 151936
    x = rng.standard_normal((rows, n)).astype(np.float32)
    x[3, 77] = x[3, 100000] = 9.0        # tie: first index wins
    dx, di, dg = dev.up(x), dev.zeros(rows * 4), dev.zeros(rows * 4)
    dev.call("m40llm_ext_argmax_f32_async", dx.ptr, rows, n, di.ptr, dg.ptr)
    dev.sync()
    idx = di.download(np.uint32, (rows,)); gap = dg.download(np.float32, (rows,))
    for r in range(rows):
        assert idx[r] == orc.sample_greedy(x[r]) == int(np.argmax(x[r]))
        srt = np.sort(x[r])
        assert gap[r] == srt[-1] - srt[-2]
    assert idx[3] == 77 and gap[3] == 0.0


def test_read_probe_xor(dev):
    # the bandwidth yardstick reads every 16-byte word exactly once: the xor over all words must match
    rng = np.random.default_rng(11)
    for n16, wgs in ((1, 1), (255, 3), (2048 * 8 + 3, 7), (700001, 512), (700001, 4096)):
        x = rng.integers(0, 2 ** 32, size=n16 * 4, dtype=np.uint32)
        dx, out = dev.up(x), dev.up(np.zeros(2048, dtype=np.uint32))
        dev.call("m40llm_ext_read_probe_async", dx.ptr, n16 * 16, wgs, out.ptr)
        dev.sync()
        assert np.bitwise_xor.reduce(out.download(np.uint32, (2048,))) == np.bitwise_xor.reduce(x)
    assert dev.lib.m40llm_ext_read_probe_async(dev.h, dx.ptr, 8, 1, out.ptr) == -2
    assert dev.lib.m40llm_ext_read_probe_async(dev.h, dx.ptr, 64, 0, out.ptr) == -2
    assert dev.lib.m40llm_ext_read_probe_async(dev.h, None, 64, 1, out.ptr) == -1


# ------------------------------------------------------------------ packed varlen prefill attention
def _prefill_call(dev, orc, q, k, v, ql, kl, qh, kvh, hd, sync_form=True, expect=0):
    dq, dk, dv = dev.up(q), dev.up(k), dev.up(v)
    dqo, dko = dev.up(orc.prefill_offsets(ql)), dev.up(orc.prefill_offsets(kl))
    dql, dkl = dev.up(np.asarray(ql, dtype=np.uint32)), dev.up(np.asarray(kl, dtype=np.uint32))
    out = dev.zeros(q.nbytes)
    name = "m40llm_attention_prefill_f32_gqa_varlen" if sync_form else "m40llm_attention_prefill_f32_gqa_varlen_async"
    dev.call(name, dq.ptr, dk.ptr, dv.ptr, dqo.ptr, dko.ptr, dql.ptr, dkl.ptr, len(ql), qh, kvh, hd, out.ptr, expect=expect)
    if not sync_form:
        dev.ctx.sync(0)
    return out.download(np.float32, q.shape)


def _modular(n, mul, mod, scale, offset):
    i = np.arange(n, dtype=np.int64)
    return ((i * mul % mod).astype(np.float32) * np.float32(scale) + np.float32(offset)).astype(np.float32)


@pytest.mark.parametrize("hd", [64, 128])
def test_prefill_varlen_reference_fixture(dev, orc, hd):
    # tests/attention_prefill_varlen.rs:93-131: (q 3, kv 3), (q 2, kv 5), (q 1, kv 4); 4 q heads, 2 kv heads
    ql, kl, qh, kvh = [3, 2, 1], [3, 5, 4], 4, 2
    q = _modular(sum(ql) * qh * hd, 17, 251, 0.0011, -0.13).reshape(sum(ql), qh, hd)
    k = _modular(sum(kl) * kvh * hd, 23, 263, 0.0009, -0.09).reshape(sum(kl), kvh, hd)
    v = _modular(sum(kl) * kvh * hd, 29, 269, 0.0013, -0.17).reshape(sum(kl), kvh, hd)
    rc, want = orc.attention_prefill(q, k, v, ql, kl, qh, kvh, hd)
    assert rc == 0
    for sync_form in (True, False):
        close(_prefill_call(dev, orc, q, k, v, ql, kl, qh, kvh, hd, sync_form), want)


@pytest.mark.parametrize("qh,kvh,hd,ql,kl", [
    (4, 2, 64, [1], [1]),                                   # one token
    (6, 2, 64, [4, 1, 7], [4, 9, 10]),                      # full prefill, one-token decode, chunked prefill
    (8, 2, 128, [70, 33, 64], [70, 97, 64]),                # query tiles with tails, key tiles with tails
    (32, 4, 64, [300, 17], [300, 529]),                     # config-1 heads, several query tiles
    (3, 3, 128, [129], [1000]),                             # 871 cached keys ahead of the queries
    (16, 2, 128, [5, 5, 5, 5, 5], [8192, 5, 37, 64, 65]),   # the longest allowed key range
    # enough long sequences (2048 queries and more) for the form of two 16-query blocks per wave -- 1088 and 1056
    # workgroups of 128 queries -- with a short sequence and cached keys ahead of the queries in the same batch
    (32, 4, 128, [2061, 2100, 50], [2161, 2100, 50]),
    (32, 4, 64, [2100, 2050, 70], [2133, 2050, 70]),
])
def test_prefill_varlen_random_vs_oracle(dev, orc, qh, kvh, hd, ql, kl):
    rng = np.random.default_rng(len(ql) + hd)
    q = rng.standard_normal((sum(ql), qh, hd)).astype(np.float32)
    k = rng.standard_normal((sum(kl), kvh, hd)).astype(np.float32)
    v = rng.standard_normal((sum(kl), kvh, hd)).astype(np.float32)
    rc, want = orc.attention_prefill(q, k, v, ql, kl, qh, kvh, hd)
    assert rc == 0
    got = _prefill_call(dev, orc, q, k, v, ql, kl, qh, kvh, hd, sync_form=False)
    close(got, want)
    # the first query of a full prefill sees one key: that V row, to what the two-part f16 split of V carries
    # (22 bits, and no finer than the f16 subnormal spacing 2^-24 for the low part)
    if ql[0] == kl[0]:
        want0 = np.repeat(v[0], qh // kvh, axis=0)
        assert np.all(np.abs(got[0] - want0) <= 2.0 ** -22 * np.abs(want0) + 2.0 ** -24)


@pytest.mark.parametrize("hd,qh,kvh", [(64, 8, 2), (128, 4, 2)])
def test_prefill_varlen_scores_rising_along_the_keys(dev, orc, hd, qh, kvh):
    # the kernel rescales its running state only when a tile holds a score well above the query's reference point: here the
    # scores rise with the key index (every tile moves the reference point; the last visible keys carry the weight), fall
    # again in a second sequence (the first tile fixes it for good), and a third holds one late key far above the rest
    rng = np.random.default_rng(hd)
    ql = kl = [700, 300, 260]
    u = rng.standard_normal(hd).astype(np.float32)
    u /= np.linalg.norm(u)
    q = (u[None, None, :] * 6.0 + 0.3 * rng.standard_normal((sum(ql), qh, hd))).astype(np.float32)
    k = (0.3 * rng.standard_normal((sum(kl), kvh, hd))).astype(np.float32)
    ramp = np.concatenate([np.arange(700) * 0.05, (300 - np.arange(300)) * 0.08, np.zeros(260)]).astype(np.float32)
    ramp[700 + 300 + 200] = 40.0
    k += ramp[:, None, None] * u[None, None, :]
    v = rng.standard_normal((sum(kl), kvh, hd)).astype(np.float32)
    rc, want = orc.attention_prefill(q, k, v, ql, kl, qh, kvh, hd)
    assert rc == 0
    got = _prefill_call(dev, orc, q, k, v, ql, kl, qh, kvh, hd, sync_form=False)
    close(got, want)
    # queries after the late key of the third sequence see (nearly) only it
    late = got[700 + 300 + 230]
    close(late, np.repeat(v[700 + 300 + 200], qh // kvh, axis=0), 1e-3, 1e-3)


def test_prefill_varlen_host_tables_form_equals_device_tables_form(dev, orc):
    # the form that validates from host copies of the tables (no read-back of the device arrays): the same bits, the same codes
    rng = np.random.default_rng(21)
    qh, kvh, hd, ql, kl = 8, 2, 128, [70, 33, 64], [70, 97, 64]
    q = rng.standard_normal((sum(ql), qh, hd)).astype(np.float32)
    k = rng.standard_normal((sum(kl), kvh, hd)).astype(np.float32)
    v = rng.standard_normal((sum(kl), kvh, hd)).astype(np.float32)
    want = _prefill_call(dev, orc, q, k, v, ql, kl, qh, kvh, hd, sync_form=False)
    dq, dk, dv = dev.up(q), dev.up(k), dev.up(v)
    h_qo, h_ko = orc.prefill_offsets(ql), orc.prefill_offsets(kl)
    h_ql, h_kl = np.asarray(ql, dtype=np.uint32), np.asarray(kl, dtype=np.uint32)
    dqo, dko, dql, dkl = dev.up(h_qo), dev.up(h_ko), dev.up(h_ql), dev.up(h_kl)
    out = dev.zeros(q.nbytes)
    name = "m40llm_ext_attention_prefill_f32_gqa_varlen_host_tables_async"
    dev.call(name, dq.ptr, dk.ptr, dv.ptr, dqo.ptr, dko.ptr, dql.ptr, dkl.ptr, h_ko.ctypes.data, h_ql.ctypes.data, h_kl.ctypes.data,
             len(ql), qh, kvh, hd, out.ptr)
    dev.ctx.sync(0)
    assert np.array_equal(out.download(np.float32, q.shape).view(np.uint32), want.view(np.uint32))
    bad = np.asarray([70, 98, 64], dtype=np.uint32)          # more queries than keys in sequence 1
    dev.call(name, dq.ptr, dk.ptr, dv.ptr, dqo.ptr, dko.ptr, dql.ptr, dkl.ptr, h_ko.ctypes.data, bad.ctypes.data, h_kl.ctypes.data,
             len(ql), qh, kvh, hd, out.ptr, expect=-8)
    dev.call(name, dq.ptr, dk.ptr, dv.ptr, dqo.ptr, dko.ptr, dql.ptr, dkl.ptr, None, h_ql.ctypes.data, h_kl.ctypes.data,
             len(ql), qh, kvh, hd, out.ptr, expect=-1)


def test_prefill_varlen_argument_checks(dev, orc):
    rng = np.random.default_rng(0)
    qh, kvh, hd, ql, kl = 4, 2, 64, [2, 3], [2, 5]
    q = rng.standard_normal((5, qh, hd)).astype(np.float32)
    k = rng.standard_normal((7, kvh, hd)).astype(np.float32)
    _prefill_call(dev, orc, q, k, k, ql, kl, qh, kvh, 32, expect=-9)
    _prefill_call(dev, orc, q, k, k, ql, kl, 5, 2, hd, expect=-3)
    _prefill_call(dev, orc, q, k, k, [2, 6], kl, qh, kvh, hd, expect=-8)       # more queries than keys
    _prefill_call(dev, orc, q, k, k, [2, 0], kl, qh, kvh, hd, expect=-8)
    _prefill_call(dev, orc, q, k, k, ql, [2, 8193], qh, kvh, hd, expect=-8)
    dq = dev.up(q)
    assert dev.lib.m40llm_attention_prefill_f32_gqa_varlen(dev.h, dq.ptr, dq.ptr, dq.ptr, dq.ptr, dq.ptr, dq.ptr, dq.ptr, 0, qh, kvh, hd, dq.ptr) == -2
    assert dev.lib.m40llm_attention_prefill_f32_gqa_varlen(dev.h, None, dq.ptr, dq.ptr, dq.ptr, dq.ptr, dq.ptr, dq.ptr, 1, qh, kvh, hd, dq.ptr) == -1
