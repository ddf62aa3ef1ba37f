"""Random-init decoder models of a given shape (synthetic weights, no checkpoint files) and their upload
through the C ABI.  Used by the parity tests and by the benchmark; tensor shapes follow the GGUF layout
the reference consumes (weights f16, [out columns][K] with K contiguous; src/infer/mapping.rs:153-203)."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import Context, check, host

TINYLLAMA_1B = dict(n_layers=22, d_model=2048, q_heads=32, kv_heads=4, head_dim=64, ffn=5632, vocab=32000,
                    rms_eps=1e-5, rope_base=10000.0, rope_scale=1.0, rope_layout=0, qkv_bias=False)
QWEN25_3B = dict(n_layers=36, d_model=2048, q_heads=16, kv_heads=2, head_dim=128, ffn=11008, vocab=151936,
                 rms_eps=1e-6, rope_base=1e6, rope_scale=1.0, rope_layout=1, qkv_bias=True)


def make_weights(cfg: dict, seed: int = 0, std: float = 0.02, emb_std: float | None = None,
                 unique_layers: int | None = None, tie_embeddings: bool = False) -> dict:
    """f16 weights ~ N(0, std), norm weights 1.0 (f32), Q/K/V biases ~ N(0, std) when cfg['qkv_bias'].
    unique_layers: draw only that many distinct layers and repeat them cyclically (throughput runs only: every
    layer still gets its own device copy, so nothing is served from a cache that a real model would miss)."""
    L, D, F, V = cfg["n_layers"], cfg["d_model"], cfg["ffn"], cfg["vocab"]
    KV = cfg["kv_heads"] * cfg["head_dim"]
    ss = np.random.SeedSequence(seed)
    streams = iter(ss.spawn(16 * L + 8))

    def w(n, k, s=std):
        rng = np.random.default_rng(next(streams))
        out = np.empty((n, k), dtype=np.float16)
        step = max(1, (1 << 24) // k)
        for i in range(0, n, step):     # bounded temporaries
            out[i:i + step] = (rng.standard_normal((min(step, n - i), k), dtype=np.float32) * np.float32(s)).astype(np.float16)
        return out.view(np.uint16)

    def b(n):
        rng = np.random.default_rng(next(streams))
        return (rng.standard_normal(n, dtype=np.float32) * np.float32(std)).astype(np.float32)

    W = dict(wq=[], wk=[], wv=[], wo=[], wgate=[], wup=[], wdown=[], attn_norm=[], ffn_norm=[])
    if cfg.get("qkv_bias"):
        W.update(bq=[], bk=[], bv=[])
    for l in range(L):
        if unique_layers and l >= unique_layers:
            for name in W:
                W[name].append(W[name][l % unique_layers])
            continue
        W["wq"].append(w(D, D)); W["wk"].append(w(KV, D)); W["wv"].append(w(KV, D)); W["wo"].append(w(D, D))
        W["wgate"].append(w(F, D)); W["wup"].append(w(F, D)); W["wdown"].append(w(D, F))
        W["attn_norm"].append(np.ones(D, dtype=np.float32)); W["ffn_norm"].append(np.ones(D, dtype=np.float32))
        if cfg.get("qkv_bias"):
            W["bq"].append(b(D)); W["bk"].append(b(KV)); W["bv"].append(b(KV))
    W["out_norm"] = np.ones(D, dtype=np.float32)
    W["lm_head"] = w(V, D)
    W["tok_emb"] = W["lm_head"] if tie_embeddings else w(V, D, emb_std if emb_std is not None else std)
    return W


class HostModelConfig(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("n_layers", "d_model", "q_heads", "kv_heads", "head_dim", "ffn", "vocab")] + \
               [(n, C.c_float) for n in ("rms_eps", "rope_base", "rope_scale")] + \
               [(n, C.c_uint32) for n in ("rope_layout", "has_qkv_bias", "norm_weight_dtype", "max_seq_len", "max_sequences")]


class HostLayerWeights(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("wq", "wk", "wv", "wo", "wgate", "wup", "wdown", "bq", "bk", "bv",
                                          "attn_norm", "ffn_norm")]


class HostKvConfig(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("mode", "recent_window", "block_size", "top_blocks", "representatives",
                                          "representative_policy", "exact_old_backing", "exact_old_attention")]


class DeviceModel:
    """Weights resident in HBM + the host-layer model object that steps through them."""

    def __init__(self, ctx: Context, cfg: dict, W: dict, max_seq_len: int, max_sequences: int = 1, kv_cfg: dict | None = None):
        self.ctx, self.cfg = ctx, cfg
        self.H = host()
        self.bufs = []
        self.weight_bytes = 0

        def up(a):
            a = np.ascontiguousarray(a)
            p = C.c_void_p()
            check(ctx.lib.m40llm_upload_weights(ctx.h, a.ctypes.data_as(C.c_void_p), a.nbytes, C.byref(p)), "m40llm_upload_weights")
            self.bufs.append(p.value)
            self.weight_bytes += a.nbytes
            return p.value

        L = cfg["n_layers"]
        layers = (HostLayerWeights * L)()
        for l in range(L):
            for name in ("wq", "wk", "wv", "wo", "wgate", "wup", "wdown", "attn_norm", "ffn_norm"):
                setattr(layers[l], name, up(W[name][l]))
            if cfg.get("qkv_bias"):
                for name in ("bq", "bk", "bv"):
                    setattr(layers[l], name, up(W[name][l]))
        self.out_norm, self.lm_head, self.tok_emb = up(W["out_norm"]), up(W["lm_head"]), up(W["tok_emb"])
        hc = HostModelConfig(cfg["n_layers"], cfg["d_model"], cfg["q_heads"], cfg["kv_heads"], cfg["head_dim"], cfg["ffn"],
                             cfg["vocab"], cfg["rms_eps"], cfg["rope_base"], cfg.get("rope_scale", 1.0), cfg["rope_layout"],
                             1 if cfg.get("qkv_bias") else 0, 1, max_seq_len, max_sequences)
        kc = None
        if kv_cfg is not None:
            kc = HostKvConfig(kv_cfg.get("mode", 2), kv_cfg["recent_window"], kv_cfg["block_size"], kv_cfg["top_blocks"], 0, 0,
                              kv_cfg.get("exact_old_backing", 2), kv_cfg.get("exact_old_attention", 2))
        self.layers = layers
        self.h = self.H.m40host_model_create(ctx.h, C.byref(hc), layers, self.out_norm, self.lm_head, self.tok_emb,
                                             C.byref(kc) if kc is not None else None)
        if not self.h:
            raise RuntimeError("m40host_model_create: " + self.H.m40host_last_error().decode())
        self.max_seq_len, self.max_sequences = max_seq_len, max_sequences

    def close(self):
        if getattr(self, "h", None):
            self.H.m40host_model_destroy(self.h)
            self.h = None
        for p in getattr(self, "bufs", []):
            self.ctx.lib.m40llm_device_free(self.ctx.h, p)
        self.bufs = []

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _ok(self, rc, what):
        if rc != 0:
            raise RuntimeError(f"{what} -> {rc}: {self.H.m40host_last_error().decode()}")

    def set_mode(self, mode: int):
        self._ok(self.H.m40host_model_set_mode(self.h, mode), "m40host_model_set_mode")

    def kv_handle(self):
        return self.H.m40host_model_kv(self.h)

    def forward_token(self, seq, pos, token, want_hidden=True, want_logits=True):
        hid = np.empty(self.cfg["d_model"], dtype=np.float32) if want_hidden else None
        log = np.empty(self.cfg["vocab"], dtype=np.float32) if want_logits else None
        self._ok(self.H.m40host_model_forward_token(self.h, seq, pos, int(token),
                                                    hid.ctypes.data_as(C.c_void_p) if want_hidden else None,
                                                    log.ctypes.data_as(C.c_void_p) if want_logits else None),
                 "m40host_model_forward_token")
        return hid, log

    def decode_greedy(self, seq, prompt, n_gen, start_pos=0):
        prompt = np.ascontiguousarray(prompt, dtype=np.uint32)
        ids = np.zeros(len(prompt) + n_gen, dtype=np.uint32)
        gaps = np.zeros(max(n_gen, 1), dtype=np.float32)
        self._ok(self.H.m40host_model_decode_greedy(self.h, seq, prompt.ctypes.data_as(C.c_void_p), len(prompt), n_gen, start_pos,
                                                    ids.ctypes.data_as(C.c_void_p), gaps.ctypes.data_as(C.c_void_p)),
                 "m40host_model_decode_greedy")
        return ids, gaps[:n_gen]

    def forward_batched(self, seq_ids, kv_lens, tokens, want_logits=True):
        s = np.ascontiguousarray(seq_ids, dtype=np.uint32); l = np.ascontiguousarray(kv_lens, dtype=np.uint32)
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        rows = len(s)
        hid = np.empty((rows, self.cfg["d_model"]), dtype=np.float32)
        log = np.empty((rows, self.cfg["vocab"]), dtype=np.float32) if want_logits else None
        self._ok(self.H.m40host_model_forward_batched(self.h, s.ctypes.data_as(C.c_void_p), l.ctypes.data_as(C.c_void_p),
                                                      t.ctypes.data_as(C.c_void_p), rows, hid.ctypes.data_as(C.c_void_p),
                                                      log.ctypes.data_as(C.c_void_p) if want_logits else None),
                 "m40host_model_forward_batched")
        return hid, log

    def decode_batch_greedy(self, seq_ids, kv_lens, first_tokens, steps):
        s = np.ascontiguousarray(seq_ids, dtype=np.uint32); l = np.ascontiguousarray(kv_lens, dtype=np.uint32)
        t = np.ascontiguousarray(first_tokens, dtype=np.uint32)
        rows = len(s)
        ids = np.zeros((rows, steps), dtype=np.uint32); gaps = np.zeros((rows, steps), dtype=np.float32)
        self._ok(self.H.m40host_model_decode_batch_greedy(self.h, s.ctypes.data_as(C.c_void_p), l.ctypes.data_as(C.c_void_p),
                                                          t.ctypes.data_as(C.c_void_p), rows, steps,
                                                          ids.ctypes.data_as(C.c_void_p), gaps.ctypes.data_as(C.c_void_p)),
                 "m40host_model_decode_batch_greedy")
        return ids, gaps

    def forward_prefill(self, seq_ids, prompts, want_logits=True):
        """Packed prefill of several prompts; returns the last token's hidden state and logits per prompt."""
        s = np.ascontiguousarray(seq_ids, dtype=np.uint32)
        lens = np.ascontiguousarray([len(p) for p in prompts], dtype=np.uint32)
        toks = np.ascontiguousarray(np.concatenate([np.asarray(p, dtype=np.uint32) for p in prompts]))
        hid = np.empty((len(s), self.cfg["d_model"]), dtype=np.float32)
        log = np.empty((len(s), self.cfg["vocab"]), dtype=np.float32) if want_logits else None
        self._ok(self.H.m40host_model_forward_prefill(self.h, s.ctypes.data_as(C.c_void_p), lens.ctypes.data_as(C.c_void_p),
                                                      toks.ctypes.data_as(C.c_void_p), len(s), hid.ctypes.data_as(C.c_void_p),
                                                      log.ctypes.data_as(C.c_void_p) if want_logits else None),
                 "m40host_model_forward_prefill")
        return hid, log

    def decode_timed(self, seq, prompt, warmup, steps):
        prompt = np.ascontiguousarray(prompt, dtype=np.uint32)
        ids = np.zeros(len(prompt) + warmup + steps, dtype=np.uint32)
        ms = C.c_double()
        self._ok(self.H.m40host_model_decode_timed(self.h, seq, prompt.ctypes.data_as(C.c_void_p), len(prompt), warmup, steps,
                                                   ids.ctypes.data_as(C.c_void_p), C.byref(ms)), "m40host_model_decode_timed")
        return ids, ms.value

    def last_timed_host_fallback(self):
        return bool(self.H.m40host_model_last_timed_host_fallback(self.h))

    def set_tie_guard(self, guard):
        self._ok(self.H.m40host_model_set_tie_guard(self.h, C.c_float(guard)), "m40host_model_set_tie_guard")

    def decode_batch_timed(self, seq_ids, kv_lens, first_tokens, warmup, steps):
        s = np.ascontiguousarray(seq_ids, dtype=np.uint32); l = np.ascontiguousarray(kv_lens, dtype=np.uint32)
        t = np.ascontiguousarray(first_tokens, dtype=np.uint32)
        ids = np.zeros((len(s), warmup + steps), dtype=np.uint32)
        ms = C.c_double()
        self._ok(self.H.m40host_model_decode_batch_timed(self.h, s.ctypes.data_as(C.c_void_p), l.ctypes.data_as(C.c_void_p),
                                                         t.ctypes.data_as(C.c_void_p), len(s), warmup, steps,
                                                         ids.ctypes.data_as(C.c_void_p), C.byref(ms)),
                 "m40host_model_decode_batch_timed")
        return ids, ms.value

    def fill_kv(self, seq, layer, k16, v16):
        """Pre-fill one (sequence, layer) slot from f16 rows [L, kv_heads, head_dim] (already rotated K)."""
        slot = self.H.m40host_model_kv_slot(self.h, seq, layer)
        dk, dv = self.ctx.to_device(k16), self.ctx.to_device(v16)
        check(self.ctx.lib.m40llm_ext_kvcache_bulk_fill_f16(self.ctx.h, self.kv_handle(), slot, dk.ptr, dv.ptr, k16.shape[0]),
              "m40llm_ext_kvcache_bulk_fill_f16")
