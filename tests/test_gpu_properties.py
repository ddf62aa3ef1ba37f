"""Size-independent properties at the full BASELINE sizes, where the oracle is too slow to be the only witness:
what the mathematics fixes whatever the kernels' decomposition into chunks, tiles and K parts."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(__file__))
from gpu_common import Dev, close, f16bits, m40  # noqa: E402

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    return Dev()


@pytest.mark.parametrize("qh,kvh,hd,L", [(32, 4, 64, 512), (16, 2, 128, 4000), (32, 8, 128, 32768)])
def test_attention_is_invariant_under_token_order(dev, qh, kvh, hd, L):
    # softmax attention without positions inside it (K arrives rotated) does not depend on the order of the cached tokens:
    # a shuffled cache must give the same output up to f32 summation order -- tokens move to other chunks, tiles and waves
    rng = np.random.default_rng(L)
    K16 = f16bits(rng.standard_normal((L, kvh, hd))).reshape(L, kvh, hd)
    V16 = f16bits(rng.standard_normal((L, kvh, hd))).reshape(L, kvh, hd)
    q = rng.standard_normal(qh * hd).astype(np.float32)
    kv = m40.KVCache(dev.ctx, L, 2, kvh, hd)
    dev.fill_dense(kv, 0, K16, V16)
    perm = rng.permutation(L)
    dev.fill_dense(kv, 1, np.ascontiguousarray(K16[perm]), np.ascontiguousarray(V16[perm]))
    a = dev.attention(kv, 0, q, qh, L)
    b = dev.attention(kv, 1, q, qh, L)
    # |out| <= max |v| ~ 4; the difference is rounding only
    assert np.abs(a - b).max() <= 2e-6, np.abs(a - b).max()
    # one distinguished token: a key aligned with the query of head 0 takes nearly all of that head's weight wherever it sits
    K2 = K16.copy().view(np.float16).astype(np.float32)
    K2[perm[0], 0] = q[:hd] * 12.0
    K2b = f16bits(K2).reshape(L, kvh, hd)
    dev.fill_dense(kv, 0, K2b, V16)
    out = dev.attention(kv, 0, q, qh, L)
    want = V16.view(np.float16).astype(np.float32)[perm[0], 0]
    score = float(np.dot(q[:hd], K2b.view(np.float16).astype(np.float32)[perm[0], 0])) / np.sqrt(hd)
    if score > 60.0:        # weight of every other token below e^-40
        close(out[:hd], want, 1e-3, 1e-4)


@pytest.mark.parametrize("M,N,K", [(1, 151936, 2048), (8, 151936, 2048), (1, 32000, 2048), (4, 14336, 4096)])
def test_projection_is_linear_in_the_activations(dev, M, N, K):
    # W (a + b) = W a + W b and W (2^k a) = 2^k W a (the second exactly: powers of two commute with every rounding here),
    # at the lm_head sizes of configs 2 and 3 and the config-4 width
    rng = np.random.default_rng(N + M)
    W = f16bits(rng.standard_normal((N, K)) * 0.02)
    a = rng.standard_normal((M, K)).astype(np.float32)
    b = rng.standard_normal((M, K)).astype(np.float32)
    ya, yb, yab = dev.gemm_gguf(a, W, M, N, K), dev.gemm_gguf(b, W, M, N, K), dev.gemm_gguf(a + b, W, M, N, K)
    scale = np.abs(a).astype(np.float64).sum(axis=1, keepdims=True) * 0.02        # ~ size of the terms of an element
    assert (np.abs(yab.astype(np.float64) - (ya.astype(np.float64) + yb.astype(np.float64))) / scale).max() <= 2e-6
    y8 = dev.gemm_gguf(a * 8.0, W, M, N, K)
    assert np.array_equal(y8, ya * 8.0)


def test_batched_attention_equals_one_call_per_sequence_config3(dev):
    # BASELINE config 3's attention: 16 q / 2 kv heads, hd 128, 8 sequences U[256, 4096] -- the row-batched launch against
    # eight single-sequence calls (src/infer/forward.rs:1930-1990 against :420-470)
    rng = np.random.default_rng(3)
    qh, kvh, hd, B, maxL = 16, 2, 128, 8, 4160
    lens = rng.integers(256, 4097, size=B).astype(np.uint32)
    ids = rng.permutation(B).astype(np.uint32)
    kv = m40.KVCache(dev.ctx, maxL, B, kvh, hd)
    for b in range(B):
        L = int(lens[b])
        dev.fill_dense(kv, int(ids[b]), f16bits(rng.standard_normal((L, kvh, hd))).reshape(L, kvh, hd),
                       f16bits(rng.standard_normal((L, kvh, hd))).reshape(L, kvh, hd))
    q = rng.standard_normal((B, qh * hd)).astype(np.float32)
    dq, out = dev.up(q), dev.zeros(q.nbytes)
    dids, dlens = dev.up(ids), dev.up(lens)
    dev.call("m40llm_attention_last_token_f32_gqa_batched_async", kv.h, dids.ptr, dlens.ptr, B, dq.ptr, qh, out.ptr)
    dev.sync()
    got = out.download(np.float32, q.shape)
    for b in range(B):
        one = dev.attention(kv, int(ids[b]), q[b], qh, int(lens[b]))
        assert np.abs(got[b] - one).max() <= 2e-6, (b, np.abs(got[b] - one).max())
