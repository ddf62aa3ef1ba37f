"""Per-element error bounds, relative to what each element is made of.

The parity tests elsewhere compare with the oracle at 1e-3 relative / 1e-4 absolute, some of them on rows scaled to a
unit maximum.  Here every element is measured against the exact (float64) value of the same inputs, in units of
S = sum_i |a_i| |w_i| -- the magnitude of the terms the element is a sum of -- so that elements with cancellation count
like any other.  Three statements per case, for the GPU result g, the oracle's f32 restatement r of the reference's
arithmetic (cuda/kernels.cu:5037-5052 for the products, :1740-1823 for the attention) and the exact value e:
  |g - e| <= 4e-7 S        (the GPU result is within a few f32 roundings of the exact value, element by element),
  max |g - e| / S <= 1.5 max |r - e| / S   (it is at least about as close to the exact value as the reference's own
                            sequential f32 sums are; measured: 2 to 30 times closer),
  |g - r| <= 1.5e-6 S      (and so the two agree element by element to that bound).
For the random inputs used S is 40-100 times the typical |element|, so 1.5e-6 S is 1.5e-4 to 6e-5 of a typical element
and far below it for the rest.
"""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(__file__))
from gpu_common import Dev, f16bits, m40  # noqa: E402

pytestmark = pytest.mark.gpu

EXACT_BOUND = 4e-7
ORACLE_BOUND = 1.5e-6


@pytest.fixture(scope="module")
def dev():
    return Dev()


def _check(label, got, oracle, exact, S):
    got = np.asarray(got, dtype=np.float64).reshape(exact.shape)
    oracle = np.asarray(oracle, dtype=np.float64).reshape(exact.shape)
    g = float((np.abs(got - exact) / S).max())
    r = float((np.abs(oracle - exact) / S).max())
    d = float((np.abs(got - oracle) / S).max())
    print(f"{label}: |gpu - exact| / S <= {g:.3e}, |oracle - exact| / S <= {r:.3e}, |gpu - oracle| / S <= {d:.3e}")
    assert g <= EXACT_BOUND, (label, g)
    assert g <= 1.5 * r, (label, g, r)
    assert d <= ORACLE_BOUND, (label, d)


@pytest.mark.parametrize("M,N,K", [(1, 5632, 2048), (1, 2048, 5632), (8, 5632, 2048), (8, 2048, 11008), (4, 4096, 4096),
                                   (300, 2048, 2048)])
def test_f16_products_per_element(dev, orc, M, N, K):
    # batch-1 GEMV, the split-K and one-launch matrix-core forms of 2-16 rows, and the many-row tiled GEMM
    rng = np.random.default_rng(M * 31 + N + K)
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = f16bits(rng.standard_normal((N, K)) * 0.02)
    W = B.view(np.float16).astype(np.float64)
    exact = A.astype(np.float64) @ W.T
    S = np.abs(A).astype(np.float64) @ np.abs(W).T
    orc.set_threads(16)
    _check(f"f32 x f16 M={M} N={N} K={K}", dev.gemm_gguf(A, B, M, N, K), orc.gemm("f32xf16_gguf", A, B, M, N, K), exact, S)


def _q80_matrix(rng, n, k):
    blob = np.empty((n, k // 32, 34), dtype=np.uint8)
    blob[:, :, :2] = rng.uniform(0.001, 0.01, size=(n, k // 32)).astype(np.float16).view(np.uint8).reshape(n, k // 32, 2)
    blob[:, :, 2:] = rng.integers(-127, 128, size=(n, k // 32, 32)).astype(np.int8).view(np.uint8)
    return blob


def _q80_values(blob):
    d = blob[:, :, :2].copy().view(np.float16).astype(np.float64)
    q = blob[:, :, 2:].view(np.int8).astype(np.float64)
    return (d * q).reshape(blob.shape[0], -1)


@pytest.mark.parametrize("N,K", [(14336, 4096), (4096, 14336)])
def test_q80_products_per_element(dev, orc, N, K):
    # BASELINE config 4 matrices: the register GEMV (1, 2 rows) and the three int8 forms -- stacked digits (3, 4 rows),
    # two operands (5, 8), three planes (9, 16) -- whose activations carry 21 signed bits per block
    rng = np.random.default_rng(N + K)
    w = _q80_matrix(rng, N, K)
    W = _q80_values(w)
    dw = dev.up(w)
    orc.set_threads(16)
    for M in (1, 2, 3, 4, 5, 8, 9, 16):
        A = rng.standard_normal((M, K)).astype(np.float32)
        exact = A.astype(np.float64) @ W.T
        S = np.abs(A).astype(np.float64) @ np.abs(W).T
        dx, dC = dev.up(A), dev.zeros(M * N * 4)
        dev.call("m40llm_ext_gemm_f32xq80_gguf_f32", dx.ptr, dw.ptr, dC.ptr, M, N, K)
        _check(f"f32 x q8_0 M={M} N={N} K={K}", dC.download(np.float32, (M, N)), orc.gemm("f32xq80_gguf", A, w, M, N, K), exact, S)


def _attention_exact(K16, V16, q, qh, kvh, hd):
    K = K16.view(np.float16).astype(np.float64)
    V = V16.view(np.float16).astype(np.float64)
    out = np.zeros((qh, hd))
    S = np.zeros((qh, hd))
    g = qh // kvh
    for h in range(qh):
        s = K[:, h // g, :] @ q.reshape(qh, hd)[h].astype(np.float64) / np.sqrt(hd)
        p = np.exp(s - s.max())
        p /= p.sum()
        out[h] = p @ V[:, h // g, :]
        S[h] = p @ np.abs(V[:, h // g, :])
    return out.reshape(-1), S.reshape(-1)


@pytest.mark.parametrize("qh,kvh,hd,L", [(32, 4, 64, 512), (32, 4, 64, 100), (16, 2, 128, 4000), (32, 8, 128, 32768)])
def test_attention_per_element(dev, orc, qh, kvh, hd, L):
    # BASELINE config 1 (one chunk, vector-ALU kernel), a short span, a config-3 row (matrix-core kernel + chunk merge) and
    # the config-5 context length dense; S = sum_t p_t |v_t|
    rng = np.random.default_rng(qh + hd + L)
    K16 = f16bits(rng.standard_normal((L, kvh, hd))).reshape(L, kvh, hd)
    V16 = f16bits(rng.standard_normal((L, kvh, hd))).reshape(L, kvh, hd)
    q = rng.standard_normal(qh * hd).astype(np.float32)
    kv = m40.KVCache(dev.ctx, L, 1, kvh, hd)
    dev.fill_dense(kv, 0, K16, V16)
    got = dev.attention(kv, 0, q, qh, L)
    orc.set_threads(16)
    oracle = orc.attention(K16[None].copy(), V16[None].copy(), L, kvh, hd, 0, q, qh, L)
    exact, S = _attention_exact(K16, V16, q, qh, kvh, hd)
    _check(f"attention qh={qh} kvh={kvh} hd={hd} L={L}", got, oracle, exact, S)
