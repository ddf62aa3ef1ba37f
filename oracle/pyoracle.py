"""ctypes view of the CPU oracle (``liboracle.so``).

TEST INFRASTRUCTURE ONLY: imported by tests, by the smoke check and by the
benchmark's CPU-baseline leg, never by the shipped path.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liboracle.so")

u32 = C.c_uint32
f32 = C.c_float
vp = C.c_void_p
sz = C.c_size_t


def build(force: bool = False) -> str:
    """Compile liboracle.so (and the reference stub witness when the reference is mounted)."""
    src = os.path.join(HERE, "oracle.c")
    stale = (not os.path.exists(LIB_PATH)) or os.path.getmtime(LIB_PATH) < max(
        os.path.getmtime(src), os.path.getmtime(os.path.join(HERE, "oracle.h")))
    if force or stale:
        subprocess.check_call(["make", "-C", HERE, "-B", "liboracle.so"])
    if os.path.exists("/root/reference/cuda/stub.c"):
        subprocess.check_call(["make", "-C", HERE, "ref"], stdout=subprocess.DEVNULL)
    return LIB_PATH


class OrcModel(C.Structure):
    _fields_ = [
        ("n_layers", u32), ("d_model", u32), ("q_heads", u32), ("kv_heads", u32),
        ("head_dim", u32), ("ffn", u32), ("vocab", u32),
        ("rms_eps", f32), ("rope_base", f32), ("rope_scale", f32),
        ("rope_layout", u32), ("has_qkv_bias", u32),
        ("wq", C.POINTER(vp)), ("wk", C.POINTER(vp)), ("wv", C.POINTER(vp)), ("wo", C.POINTER(vp)),
        ("wgate", C.POINTER(vp)), ("wup", C.POINTER(vp)), ("wdown", C.POINTER(vp)),
        ("bq", C.POINTER(vp)), ("bk", C.POINTER(vp)), ("bv", C.POINTER(vp)),
        ("attn_norm", C.POINTER(vp)), ("ffn_norm", C.POINTER(vp)),
        ("out_norm", vp), ("lm_head", vp), ("tok_emb", vp),
    ]


class OrcCkv(C.Structure):
    _fields_ = [
        ("max_seq_len", u32), ("max_batch", u32), ("kv_heads", u32), ("head_dim", u32),
        ("recent_window", u32), ("block_size", u32),
        ("recent_k", vp), ("recent_v", vp), ("old_k", vp), ("q4_v", vp), ("q4_scale", vp),
        ("seq_map", vp), ("v_format", u32), ("q4_dm", vp),
    ]


class OrcModelKv(C.Structure):
    _fields_ = [("max_seq_len", u32), ("max_sequences", u32), ("K", vp), ("V", vp)]


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        build()
    L = C.CDLL(LIB_PATH)

    def sig(name, res, *args):
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = list(args)

    sig("orc_f32_to_f16", C.c_uint16, f32)
    sig("orc_f16_to_f32", f32, C.c_uint16)
    sig("orc_f32_to_f16_n", None, vp, vp, sz)
    sig("orc_f16_to_f32_n", None, vp, vp, sz)
    sig("orc_kv_elems_per_token", sz, u32, u32)
    sig("orc_kv_base", sz, u32, u32, u32, u32, u32)
    sig("orc_kv_index", sz, u32, u32, u32, u32, u32, u32, u32)
    sig("orc_rms_norm", None, vp, vp, u32, u32, f32)
    sig("orc_rms_norm_weighted", C.c_int, vp, vp, vp, u32, u32, f32, u32)
    sig("orc_rope_inplace", None, vp, u32, u32, u32, u32, f32, f32, u32)
    sig("orc_residual_add", None, vp, vp, vp, sz)
    sig("orc_swiglu", None, vp, vp, vp, sz)
    sig("orc_q80_to_f32", None, vp, vp, sz)
    for n in ("orc_gemm_f32xf16_gguf", "orc_gemm_f32xf16_rowmajor", "orc_gemm_f16xf16_rowmajor",
              "orc_gemm_f32xq80_gguf"):
        sig(n, None, vp, vp, vp, C.c_int, C.c_int, C.c_int)
    sig("orc_ffn_swiglu_q80", None, vp, vp, vp, vp, vp, vp, vp, C.c_int, C.c_int, C.c_int)
    sig("orc_kv_append_f32", None, vp, vp, u32, u32, u32, u32, u32, vp, vp)
    sig("orc_kv_append_f32_rope_k", None, vp, vp, u32, u32, u32, u32, u32, vp, vp, f32, f32, u32)
    sig("orc_attention_last_token_gqa", None, vp, vp, u32, u32, u32, u32, vp, u32, u32, vp)
    sig("orc_attention_last_token_gqa_batched", None, vp, vp, u32, u32, u32, vp, vp, u32, vp, u32, vp)
    sig("orc_attention_prefill_gqa_varlen", C.c_int, vp, vp, vp, vp, vp, vp, vp, u32, u32, u32, u32, vp)
    sig("orc_inv_sqrt_head_dim", f32, u32)
    sig("orc_ckv_create", C.POINTER(OrcCkv), u32, u32, u32, u32, u32, u32)
    sig("orc_ckv_destroy", None, C.POINTER(OrcCkv))
    sig("orc_ckv_bytes_old_k", sz, C.POINTER(OrcCkv))
    sig("orc_ckv_bytes_q4_v", sz, C.POINTER(OrcCkv))
    sig("orc_ckv_bytes_q4_scale", sz, C.POINTER(OrcCkv))
    sig("orc_ckv_create_fmt", C.POINTER(OrcCkv), u32, u32, u32, u32, u32, u32, u32)
    sig("orc_q4g32_quantize_row", None, vp, u32, vp, vp)
    sig("orc_q4g32_unpack", f32, C.c_uint8, u32, u32)
    sig("orc_q4_quantize_row", None, vp, u32, vp, vp)
    sig("orc_q4_unpack", f32, C.c_uint8, u32, f32)
    sig("orc_ckv_append_rope_k_at", C.c_int, C.POINTER(OrcCkv), u32, u32, vp, vp, f32, f32, u32)
    sig("orc_ckv_block_scores", u32, C.POINTER(OrcCkv), u32, vp, u32, u32, u32, u32, C.c_int, vp, vp)
    sig("orc_select_top_blocks", u32, vp, u32, u32, vp, vp)
    sig("orc_ckv_attention_block_select", C.c_int, C.POINTER(OrcCkv), u32, vp, u32, u32, u32, u32,
        u32, C.c_int, vp, vp, vp)
    sig("orc_dense_attention_block_select", C.c_int, vp, vp, u32, u32, u32, u32, vp, u32, u32, u32,
        u32, u32, C.c_int, vp, vp, vp)
    sig("orc_ckv_debug_select_old_blocks", C.c_int, C.POINTER(OrcCkv), u32, vp, u32, u32, vp, vp,
        vp, vp, vp, u32, vp)
    sig("orc_greedy_topk1", u32, vp, sz)
    sig("orc_sample_greedy", u32, vp, sz)
    sig("orc_top2_gap", f32, vp, sz)
    sig("orc_model_kv_create", C.POINTER(OrcModelKv), C.POINTER(OrcModel), u32, u32)
    sig("orc_model_kv_destroy", None, C.POINTER(OrcModelKv))
    sig("orc_layer_forward", None, C.POINTER(OrcModel), C.POINTER(OrcModelKv), u32, u32, u32, vp, vp)
    sig("orc_token_forward", None, C.POINTER(OrcModel), C.POINTER(OrcModelKv), u32, u32, u32, vp)
    sig("orc_prefill_forward", C.c_int, C.POINTER(OrcModel), C.POINTER(OrcModelKv), vp, vp, vp, u32, vp)
    sig("orc_logits", None, C.POINTER(OrcModel), vp, vp)
    sig("orc_decode_greedy", None, C.POINTER(OrcModel), C.POINTER(OrcModelKv), u32, vp, u32, u32,
        u32, vp, vp)
    sig("orc_set_threads", None, C.c_int)
    sig("orc_get_threads", C.c_int)
    _lib = L
    return L


def ptr(a: np.ndarray | None):
    """Raw pointer of a C-contiguous numpy array (None -> NULL)."""
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"], "oracle needs C-contiguous arrays"
    return a.ctypes.data_as(vp)


# ---------------------------------------------------------------------------
# Convenience wrappers (numpy in, numpy out)
# ---------------------------------------------------------------------------

def f32_to_f16_bits(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().orc_f32_to_f16_n(ptr(x), ptr(out), x.size)
    return out


def f16_bits_to_f32(h: np.ndarray) -> np.ndarray:
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, dtype=np.float32)
    lib().orc_f16_to_f32_n(ptr(h), ptr(out), h.size)
    return out


def rms_norm(x, eps, weight=None, weight_dtype=1):
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, dim = x.shape
    out = np.empty_like(x)
    if weight is None:
        lib().orc_rms_norm(ptr(x), ptr(out), rows, dim, eps)
    else:
        w = np.ascontiguousarray(weight)
        rc = lib().orc_rms_norm_weighted(ptr(x), ptr(w), ptr(out), rows, dim, eps, weight_dtype)
        assert rc == 0, rc
    return out


def rope(x, num_heads, head_dim, past_len, base, scale, layout):
    x = np.array(x, dtype=np.float32, order="C", copy=True)
    rows = x.shape[0]
    lib().orc_rope_inplace(ptr(x), rows, num_heads, head_dim, past_len, base, scale, layout)
    return x


def swiglu(g, u):
    g = np.ascontiguousarray(g, dtype=np.float32)
    u = np.ascontiguousarray(u, dtype=np.float32)
    out = np.empty_like(g)
    lib().orc_swiglu(ptr(g), ptr(u), ptr(out), g.size)
    return out


def residual_add(a, b):
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    out = np.empty_like(a)
    lib().orc_residual_add(ptr(a), ptr(b), ptr(out), a.size)
    return out


def q80_to_f32(blocks: np.ndarray, n: int) -> np.ndarray:
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    out = np.empty(n, dtype=np.float32)
    lib().orc_q80_to_f32(ptr(blocks), ptr(out), n)
    return out


def gemm(kind: str, A, B, M, N, K) -> np.ndarray:
    """kind in {'f32xf16_gguf','f32xf16_rowmajor','f16xf16_rowmajor','f32xq80_gguf'}"""
    A = np.ascontiguousarray(A)
    B = np.ascontiguousarray(B)
    out = np.empty((M, N), dtype=np.float32)
    getattr(lib(), "orc_gemm_" + kind)(ptr(A), ptr(B), ptr(out), M, N, K)
    return out


def ffn_swiglu_q80(x, wg, wu, wd, M, d_model, ffn):
    x = np.ascontiguousarray(x, dtype=np.float32)
    sg = np.empty((M, ffn), dtype=np.float32)
    su = np.empty((M, ffn), dtype=np.float32)
    out = np.empty((M, d_model), dtype=np.float32)
    lib().orc_ffn_swiglu_q80(ptr(x), ptr(wg), ptr(wu), ptr(wd), ptr(sg), ptr(su), ptr(out), M, d_model, ffn)
    return out


def attention(K, V, max_seq_len, kv_heads, head_dim, seq, q, q_heads, seq_len):
    q = np.ascontiguousarray(q, dtype=np.float32)
    out = np.zeros(q_heads * head_dim, dtype=np.float32)
    lib().orc_attention_last_token_gqa(ptr(K), ptr(V), max_seq_len, kv_heads, head_dim, seq,
                                       ptr(q), q_heads, seq_len, ptr(out))
    return out


def prefill_offsets(lens):
    """exclusive prefix of token counts (u32), as the reference's batch metadata builds it (src/infer/batch.rs:276-355)"""
    lens = np.asarray(lens, dtype=np.uint32)
    return np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.uint32)


def attention_prefill(q, k, v, q_lens, kv_lens, q_heads, kv_heads, head_dim):
    """q [total_q, q_heads, hd], k/v [total_kv, kv_heads, hd], all f32 -> (rc, out like q)"""
    q = np.ascontiguousarray(q, dtype=np.float32); k = np.ascontiguousarray(k, dtype=np.float32)
    v = np.ascontiguousarray(v, dtype=np.float32)
    ql = np.ascontiguousarray(q_lens, dtype=np.uint32); kl = np.ascontiguousarray(kv_lens, dtype=np.uint32)
    qo, ko = prefill_offsets(ql), prefill_offsets(kl)
    out = np.zeros_like(q)
    rc = lib().orc_attention_prefill_gqa_varlen(ptr(q), ptr(k), ptr(v), ptr(qo), ptr(ko), ptr(ql), ptr(kl), len(ql),
                                                q_heads, kv_heads, head_dim, ptr(out))
    return rc, out


def attention_batched(K, V, max_seq_len, kv_heads, head_dim, seq_ids, seq_lens, q, q_heads):
    ids = np.ascontiguousarray(seq_ids, dtype=np.uint32)
    lens = np.ascontiguousarray(seq_lens, dtype=np.uint32)
    q = np.ascontiguousarray(q, dtype=np.float32)
    out = np.zeros(q.shape, dtype=np.float32)
    lib().orc_attention_last_token_gqa_batched(ptr(K), ptr(V), max_seq_len, kv_heads, head_dim,
                                               ptr(ids), ptr(lens), len(ids), ptr(q), q_heads, ptr(out))
    return out


class CompressedKV:
    """fp16-K / q4-V compressed cache model (one object = all sequences)."""

    def __init__(self, max_seq_len, max_batch, kv_heads, head_dim, recent_window, block_size, v_format=0):
        """v_format 0: the reference's q4 V (one f32 scale per token and head); 1: groups of 32, f16 scale + f16 min."""
        self.p = lib().orc_ckv_create_fmt(max_seq_len, max_batch, kv_heads, head_dim, recent_window, block_size, v_format)
        assert self.p, "orc_ckv_create failed"
        self.v_format = v_format
        self.max_seq_len, self.max_batch = max_seq_len, max_batch
        self.kv_heads, self.head_dim = kv_heads, head_dim
        self.recent_window, self.block_size = recent_window, block_size

    def __del__(self):
        if getattr(self, "p", None):
            lib().orc_ckv_destroy(self.p)
            self.p = None

    def _view(self, field, dtype, shape):
        addr = getattr(self.p.contents, field)
        n = int(np.prod(shape))
        buf = (C.c_char * (n * np.dtype(dtype).itemsize)).from_address(addr)
        return np.frombuffer(buf, dtype=dtype).reshape(shape)

    @property
    def recent_k(self):
        return self._view("recent_k", np.uint16, (self.max_batch, self.recent_window, self.kv_heads, self.head_dim))

    @property
    def recent_v(self):
        return self._view("recent_v", np.uint16, (self.max_batch, self.recent_window, self.kv_heads, self.head_dim))

    @property
    def old_k(self):
        return self._view("old_k", np.uint16, (self.max_batch, self.max_seq_len, self.kv_heads, self.head_dim))

    @property
    def q4_v(self):
        return self._view("q4_v", np.uint8, (self.max_batch, self.max_seq_len, self.kv_heads, self.head_dim // 2))

    @property
    def q4_scale(self):
        return self._view("q4_scale", np.float32, (self.max_batch, self.max_seq_len, self.kv_heads))

    @property
    def q4_dm(self):
        return self._view("q4_dm", np.uint32, (self.max_batch, self.max_seq_len, self.kv_heads, self.head_dim // 32))

    @property
    def seq_map(self):
        return self._view("seq_map", np.uint32, (self.max_batch,))

    def bytes(self):
        L = lib()
        return (L.orc_ckv_bytes_old_k(self.p), L.orc_ckv_bytes_q4_v(self.p), L.orc_ckv_bytes_q4_scale(self.p))

    def append(self, seq, position, k, v, base=10000.0, scale=1.0, layout=0):
        k = np.ascontiguousarray(k, dtype=np.float32)
        v = np.ascontiguousarray(v, dtype=np.float32)
        return lib().orc_ckv_append_rope_k_at(self.p, seq, position, ptr(k), ptr(v), base, scale, layout)

    def bulk_fill(self, seq, k_f16_bits, v_f16_bits):
        """Fill positions 0..L-1 from already-rotated f16 K / f16 V, exactly as L ordered appends would."""
        L = k_f16_bits.shape[0]
        W = self.recent_window
        old_len = max(L - W, 0)
        if old_len:
            self.old_k[seq, :old_len] = k_f16_bits[:old_len]
            packed = np.empty(self.head_dim // 2, dtype=np.uint8)
            sc = np.empty(1, dtype=np.float32)
            dm = np.empty(self.head_dim // 32, dtype=np.uint32)
            for t in range(old_len):
                for h in range(self.kv_heads):
                    row = np.ascontiguousarray(v_f16_bits[t, h])
                    if self.v_format:
                        lib().orc_q4g32_quantize_row(ptr(row), self.head_dim, ptr(packed), ptr(dm))
                        self.q4_dm[seq, t, h] = dm
                    else:
                        lib().orc_q4_quantize_row(ptr(row), self.head_dim, ptr(packed), ptr(sc))
                        self.q4_scale[seq, t, h] = sc[0]
                    self.q4_v[seq, t, h] = packed
        for t in range(old_len, L):
            self.recent_k[seq, t % W] = k_f16_bits[t]
            self.recent_v[seq, t % W] = v_f16_bits[t]
        self.seq_map[seq] = L

    def block_scores(self, seq, q_head, kv_head, seq_len, order, recent_window=None, block_size=None):
        W = recent_window or self.recent_window
        bs = block_size or self.block_size
        old_len = max(seq_len - W, 0)
        nblk = (old_len + bs - 1) // bs if old_len else 0
        q_head = np.ascontiguousarray(q_head, dtype=np.float32)
        out = np.zeros(max(nblk, 1), dtype=np.float32)
        out64 = np.zeros(max(nblk, 1), dtype=np.float64)
        n = lib().orc_ckv_block_scores(self.p, seq, ptr(q_head), kv_head, seq_len, W, bs, order,
                                       ptr(out), ptr(out64))
        return (out64[:n] if order == 1 else out[:n])

    def attention(self, seq, q, q_heads, seq_len, top_blocks, score_order=2, recent_window=None,
                  block_size=None):
        W = recent_window or self.recent_window
        bs = block_size or self.block_size
        q = np.ascontiguousarray(q, dtype=np.float32)
        out = np.zeros(q_heads * self.head_dim, dtype=np.float32)
        sel = np.full((q_heads, 64), 0xFFFFFFFF, dtype=np.uint32)
        cnt = np.zeros(q_heads, dtype=np.uint32)
        rc = lib().orc_ckv_attention_block_select(self.p, seq, ptr(q), q_heads, seq_len, W, bs,
                                                  top_blocks, score_order, ptr(out), ptr(sel), ptr(cnt))
        return rc, out, sel, cnt

    def debug_select(self, seq, q_head0, seq_len, top_blocks, max_out=2048):
        q_head0 = np.ascontiguousarray(q_head0, dtype=np.float32)
        blocks = np.zeros(max_out, dtype=np.uint32)
        scores = np.zeros(max_out, dtype=np.float32)
        start = np.zeros(max_out, dtype=np.uint32)
        end = np.zeros(max_out, dtype=np.uint32)
        count = np.zeros(1, dtype=np.uint32)
        total = np.zeros(1, dtype=np.uint32)
        rc = lib().orc_ckv_debug_select_old_blocks(self.p, seq, ptr(q_head0), seq_len, top_blocks,
                                                   ptr(blocks), ptr(scores), ptr(start), ptr(end),
                                                   ptr(count), max_out, ptr(total))
        n = int(count[0])
        return rc, blocks[:n], scores[:n], start[:n], end[:n], int(total[0])


def dense_block_select(K, V, max_seq_len, kv_heads, head_dim, seq, q, q_heads, seq_len, W, bs, top,
                       score_order=2):
    q = np.ascontiguousarray(q, dtype=np.float32)
    out = np.zeros(q_heads * head_dim, dtype=np.float32)
    sel = np.full((q_heads, 64), 0xFFFFFFFF, dtype=np.uint32)
    cnt = np.zeros(q_heads, dtype=np.uint32)
    rc = lib().orc_dense_attention_block_select(ptr(K), ptr(V), max_seq_len, kv_heads, head_dim, seq,
                                                ptr(q), q_heads, seq_len, W, bs, top, score_order,
                                                ptr(out), ptr(sel), ptr(cnt))
    return rc, out, sel, cnt


def select_top_blocks(scores, top_blocks):
    scores = np.ascontiguousarray(scores, dtype=np.float32)
    ob = np.zeros(64, dtype=np.uint32)
    os_ = np.zeros(64, dtype=np.float32)
    n = lib().orc_select_top_blocks(ptr(scores), len(scores), top_blocks, ptr(ob), ptr(os_))
    return ob[:n], os_[:n]


def greedy_topk1(logits):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    return int(lib().orc_greedy_topk1(ptr(logits), logits.size))


def sample_greedy(logits):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    return int(lib().orc_sample_greedy(ptr(logits), logits.size))


class Model:
    """Holds numpy weights alive and exposes them to the C oracle as an ``orc_model``."""

    def __init__(self, cfg: dict, weights: dict):
        self.cfg = cfg
        self.w = weights  # keeps arrays alive
        nl = cfg["n_layers"]
        m = OrcModel()
        for k in ("n_layers", "d_model", "q_heads", "kv_heads", "head_dim", "ffn", "vocab", "rope_layout"):
            setattr(m, k, cfg[k])
        m.rms_eps = cfg["rms_eps"]
        m.rope_base = cfg["rope_base"]
        m.rope_scale = cfg.get("rope_scale", 1.0)
        m.has_qkv_bias = 1 if cfg.get("qkv_bias") else 0
        self._arrays = []

        def table(name):
            arr = (vp * nl)()
            for l in range(nl):
                a = weights[name][l]
                assert a.flags["C_CONTIGUOUS"]
                arr[l] = a.ctypes.data
            self._arrays.append(arr)
            return C.cast(arr, C.POINTER(vp))

        for name in ("wq", "wk", "wv", "wo", "wgate", "wup", "wdown", "attn_norm", "ffn_norm"):
            setattr(m, name, table(name))
        if m.has_qkv_bias:
            for name in ("bq", "bk", "bv"):
                setattr(m, name, table(name))
        m.out_norm = weights["out_norm"].ctypes.data
        m.lm_head = weights["lm_head"].ctypes.data
        m.tok_emb = weights["tok_emb"].ctypes.data
        self.m = m
        self.kv = None

    def alloc_kv(self, max_seq_len, max_sequences=1):
        if self.kv:
            lib().orc_model_kv_destroy(self.kv)
        self.kv = lib().orc_model_kv_create(C.byref(self.m), max_seq_len, max_sequences)
        assert self.kv, "oracle KV allocation failed"
        self.max_seq_len, self.max_sequences = max_seq_len, max_sequences

    def kv_views(self):
        c = self.cfg
        shape = (self.max_sequences * c["n_layers"], self.max_seq_len, c["kv_heads"], c["head_dim"])
        n = int(np.prod(shape))
        K = np.frombuffer((C.c_char * (2 * n)).from_address(self.kv.contents.K), dtype=np.uint16).reshape(shape)
        V = np.frombuffer((C.c_char * (2 * n)).from_address(self.kv.contents.V), dtype=np.uint16).reshape(shape)
        return K, V

    def layer_forward(self, layer, seq, pos, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.empty_like(x)
        lib().orc_layer_forward(C.byref(self.m), self.kv, layer, seq, pos, ptr(x), ptr(out))
        return out

    def token_forward(self, seq, pos, token_id):
        out = np.empty(self.cfg["d_model"], dtype=np.float32)
        lib().orc_token_forward(C.byref(self.m), self.kv, seq, pos, int(token_id), ptr(out))
        return out

    def prefill_forward(self, seq_ids, prompts):
        """Packed prefill of several prompts (each from position 0 of its sequence): hidden rows [sum of lens][d_model]."""
        ids = np.ascontiguousarray(seq_ids, dtype=np.uint32)
        lens = np.ascontiguousarray([len(p) for p in prompts], dtype=np.uint32)
        toks = np.ascontiguousarray(np.concatenate([np.asarray(p, dtype=np.uint32) for p in prompts]))
        out = np.empty((int(lens.sum()), self.cfg["d_model"]), dtype=np.float32)
        rc = lib().orc_prefill_forward(C.byref(self.m), self.kv, ptr(ids), ptr(lens), ptr(toks), len(ids), ptr(out))
        assert rc == 0, rc
        return out

    def logits(self, hidden):
        hidden = np.ascontiguousarray(hidden, dtype=np.float32)
        out = np.empty(self.cfg["vocab"], dtype=np.float32)
        lib().orc_logits(C.byref(self.m), ptr(hidden), ptr(out))
        return out

    def decode_greedy(self, seq, prompt, n_gen, start_pos=0):
        prompt = np.ascontiguousarray(prompt, dtype=np.uint32)
        ids = np.zeros(len(prompt) + n_gen, dtype=np.uint32)
        gaps = np.zeros(max(n_gen, 1), dtype=np.float32)
        lib().orc_decode_greedy(C.byref(self.m), self.kv, seq, ptr(prompt), len(prompt), n_gen,
                                start_pos, ptr(ids), ptr(gaps))
        return ids, gaps[:n_gen]

    def __del__(self):
        if getattr(self, "kv", None):
            lib().orc_model_kv_destroy(self.kv)
            self.kv = None


def set_threads(n: int):
    lib().orc_set_threads(int(n))
