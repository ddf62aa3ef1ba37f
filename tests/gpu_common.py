"""Helpers shared by the GPU parity tests: everything goes through the C-ABI library."""
import ctypes as C
import importlib

import numpy as np

m40 = importlib.import_module("m40-llm_amd")

RTOL, ATOL = 1e-3, 1e-4   # float parity bar of the hot path: 1e-3 relative / 1e-4 absolute


def close(got, want, rtol=RTOL, atol=ATOL):
    got = np.asarray(got, dtype=np.float64); want = np.asarray(want, dtype=np.float64)
    err = np.abs(got - want)
    ok = err <= atol + rtol * np.abs(want)
    if not ok.all():
        i = int(np.argmax(err - (atol + rtol * np.abs(want))))
        raise AssertionError(f"mismatch at flat index {i}: got {got.flat[i]!r} want {want.flat[i]!r} "
                             f"(max abs err {err.max():.3e}, {int((~ok).sum())}/{ok.size} outside tolerance)")
    return True


def f16bits(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32).astype(np.float16).view(np.uint16))


class Dev:
    """One context + convenience calls; every compute call is a single m40llm_* symbol."""

    def __init__(self):
        self.ctx = m40.Context(0)
        self.lib = self.ctx.lib
        self.h = self.ctx.h

    def up(self, a):
        return self.ctx.to_device(np.ascontiguousarray(a))

    def zeros(self, nbytes):
        return self.up(np.zeros(max(nbytes, 1), dtype=np.uint8))

    def call(self, name, *args, expect=0):
        rc = getattr(self.lib, name)(self.h, *args)
        assert rc == expect, f"{name} returned {rc}, expected {expect}"
        return rc

    def sync(self):
        self.ctx.sync(0); self.ctx.sync(1)

    def gemm_gguf(self, A, B16, M, N, K):
        dA, dB = self.up(A), self.up(B16)
        dC = self.zeros(M * N * 4)
        self.call("m40llm_gemm_f32xf16_gguf_f32", dA.ptr, dB.ptr, dC.ptr, M, N, K)
        return dC.download(np.float32, (M, N))

    def fill_dense(self, kv, seq, K16, V16):
        """K16/V16: [L, kvh, hd] uint16"""
        dk, dv = self.up(K16), self.up(V16)
        self.call("m40llm_ext_kvcache_bulk_fill_f16", kv.h, seq, dk.ptr, dv.ptr, K16.shape[0])

    def attention(self, kv, seq, q, q_heads, seq_len):
        dq = self.up(np.asarray(q, dtype=np.float32))
        out = self.zeros(q_heads * kv.head_dim * 4)
        self.call("m40llm_attention_last_token_f32_gqa_async", kv.h, seq, dq.ptr, q_heads, seq_len, out.ptr)
        self.ctx.sync(1)
        return out.download(np.float32, (q_heads * kv.head_dim,))
