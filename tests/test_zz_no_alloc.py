"""The entry point that allocates nothing: m40llm_ext_attention_last_token_f32_gqa_static_scratch_async.

Its chunk partials live in a fixed device array inside the library instead of the context's arena.  Checked against
the allocating entry point it is a variant of (same kernels and chunking: results must be bit-identical, which is
inside the 1e-3 / 1e-4 float bar) and against the oracle, on two calls in a row, the second with a smaller input that
leaves stale partials of the first call in the shared array.
"""
import numpy as np
import pytest

from gpu_common import Dev, close, f16bits, m40

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    return Dev()


def _case(dev, orc, qh, kvh, hd, lengths, seed):
    rng = np.random.default_rng(seed)
    Lmax = max(lengths)
    k16 = f16bits(rng.standard_normal((Lmax, kvh, hd)))
    v16 = f16bits(rng.standard_normal((Lmax, kvh, hd)))
    kv = m40.KVCache(dev.ctx, Lmax, 1, kvh, hd)
    dev.fill_dense(kv, 0, k16, v16)
    for L in lengths:                      # consecutive calls on the same GPU share the fixed array
        q = rng.standard_normal(qh * hd).astype(np.float32)
        dq = dev.up(q)
        out_static, out_arena = dev.zeros(qh * hd * 4), dev.zeros(qh * hd * 4)
        dev.call("m40llm_ext_attention_last_token_f32_gqa_static_scratch_async", kv.h, 0, dq.ptr, qh, L, out_static.ptr)
        dev.call("m40llm_attention_last_token_f32_gqa_async", kv.h, 0, dq.ptr, qh, L, out_arena.ptr)
        dev.sync()
        got = out_static.download(np.float32, (qh * hd,))
        ref = out_arena.download(np.float32, (qh * hd,))
        assert np.array_equal(got, ref), (L, float(np.abs(got - ref).max()))
        want = orc.attention(np.ascontiguousarray(k16[None]), np.ascontiguousarray(v16[None]), Lmax, kvh, hd, 0, q, qh, L)
        close(got, want)
    kv.destroy()


def test_static_scratch_two_calls_second_smaller(dev, orc):
    # 9000 tokens: several chunks and the merge launch; then 1500 (fewer chunks over the stale partials), then a
    # one-chunk row that does not touch the array at all
    _case(dev, orc, 32, 8, 128, [9000, 1500, 300], seed=0)
    _case(dev, orc, 32, 4, 64, [4096, 700], seed=1)


def test_static_scratch_argument_codes_and_size_limit(dev):
    qh, kvh, hd = 32, 4, 64
    kv = m40.KVCache(dev.ctx, 64, 1, kvh, hd)
    dq, out = dev.zeros(qh * hd * 4), dev.zeros(qh * hd * 4)
    name = "m40llm_ext_attention_last_token_f32_gqa_static_scratch_async"
    dev.call(name, kv.h, 1, dq.ptr, qh, 8, out.ptr, expect=-2)
    dev.call(name, kv.h, 0, dq.ptr, qh, 0, out.ptr, expect=-3)
    dev.call(name, kv.h, 0, dq.ptr, qh, 65, out.ptr, expect=-3)
    dev.call(name, kv.h, 0, dq.ptr, qh + 1, 8, out.ptr, expect=-6)
    kv.destroy()
    # 128 q heads x 64 chunks x 66 floats = 2.06 MiB of partials: beyond the fixed 2 MiB, refused before any launch
    qh = kvh = 128
    L = 131072
    big = m40.KVCache(dev.ctx, L, 1, kvh, hd)
    dq, out = dev.zeros(qh * hd * 4), dev.zeros(qh * hd * 4)
    dev.call(name, big.h, 0, dq.ptr, qh, L, out.ptr, expect=-9)
    dev.call(name, big.h, 0, dq.ptr, qh, L // 2, out.ptr)      # half the chunks fit
    dev.sync()
    big.destroy()


def test_static_scratch_second_context_is_refused_while_busy(dev, orc):
    """The fixed array is one per GPU: a call from another context while the last user's launches are still outstanding
    returns -10 (busy) instead of racing; once that work has finished the call goes through and gives the arena path's
    bits."""
    qh, kvh, hd, L = 64, 8, 128, 60000
    rng = np.random.default_rng(5)
    k16 = f16bits(rng.standard_normal((L, kvh, hd), dtype=np.float32))
    v16 = f16bits(rng.standard_normal((L, kvh, hd), dtype=np.float32))
    name = "m40llm_ext_attention_last_token_f32_gqa_static_scratch_async"
    other = Dev()
    kv1, kv2 = m40.KVCache(dev.ctx, L, 1, kvh, hd), m40.KVCache(other.ctx, L, 1, kvh, hd)
    dev.fill_dense(kv1, 0, k16, v16); other.fill_dense(kv2, 0, k16, v16)
    q = rng.standard_normal(qh * hd).astype(np.float32)
    dq1, dq2 = dev.up(q), other.up(q)
    o1, o2, o3 = dev.zeros(qh * hd * 4), other.zeros(qh * hd * 4), other.zeros(qh * hd * 4)
    dev.sync(); other.sync()
    for _ in range(4):                      # a few launches in a row keep the first context's stream busy
        dev.call(name, kv1.h, 0, dq1.ptr, qh, L, o1.ptr)
    rc = getattr(other.lib, name)(other.h, kv2.h, 0, dq2.ptr, qh, L, o2.ptr)
    assert rc in (0, -10), rc
    dev.sync(); other.sync()
    other.call(name, kv2.h, 0, dq2.ptr, qh, L, o2.ptr)
    other.call("m40llm_attention_last_token_f32_gqa_async", kv2.h, 0, dq2.ptr, qh, L, o3.ptr)
    other.sync()
    got = o2.download(np.float32, (qh * hd,))
    assert np.array_equal(got, o3.download(np.float32, (qh * hd,)))
    assert np.array_equal(got, o1.download(np.float32, (qh * hd,)))
    print(f"[static scratch] second context while busy returned {rc}")
    kv1.destroy(); kv2.destroy()
