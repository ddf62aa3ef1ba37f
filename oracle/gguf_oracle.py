"""CPU restatement of the reference's GGUF ingestion: file parser, tensor views, model configuration from
metadata, tensor-name mapping, lm_head / tied-embedding rules and the embedding-row load.

TEST INFRASTRUCTURE ONLY.  Nothing in the product imports this module; the tests use it as the checker for
the C++ host layer (m40-llm_amd/host/gguf.hpp) and for the device loader.

Each function cites the reference code it follows.  Errors are raised as GgufError with the reference's
message text (the reference's tests match on substrings of those messages).

Pins (tests/test_gguf.py): every literal case of the reference's tests/gguf_metadata_config.rs,
tests/gguf_device_views.rs, tests/gguf_device_views_offsets.rs, tests/model_config_parsing.rs,
tests/infer_metadata_validation.rs, tests/map_standard_layer.rs (mapping cases) and
tests/embedding_dequant_cuda.rs, rebuilt byte for byte with an independent writer; the q8_0 row dequant
against the q8_0 block pins of oracle.c (orc_q80_to_f32).
"""
from __future__ import annotations

import struct

import numpy as np


class GgufError(ValueError):
    pass


# GGUF metadata value types (src/gguf.rs:14-53)
U8, I8, U16, I16, U32, I32, F32, BOOL, STR, ARRAY, U64, I64, F64 = range(13)
_SCALAR_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", U64: "<Q", I64: "<q", F64: "<d"}

# ggml dtype codes (src/gguf.rs:110-131) and their (elements per block, bytes per block)
# (src/gguf.rs:305-322, src/infer/meta.rs:156-223)
DTYPE_NAMES = {0: "F32", 1: "F16", 2: "Q4_0", 3: "Q4_1", 6: "Q5_0", 7: "Q5_1", 8: "Q8_0", 9: "Q8_1", 10: "Q2K",
               11: "Q3K", 12: "Q4K", 13: "Q5K", 14: "Q6K", 15: "Q8K"}
DTYPE_LAYOUT = {"F32": (1, 4), "F16": (1, 2), "Q4_0": (32, 18), "Q4_1": (32, 20), "Q5_0": (32, 22), "Q5_1": (32, 36),
                "Q8_0": (32, 34), "Q8_1": (32, 36), "Q2K": (256, 84), "Q3K": (256, 110), "Q4K": (256, 144),
                "Q5K": (256, 176), "Q6K": (256, 210), "Q8K": (256, 292)}

EMBEDDING_NAMES = ["tok_embeddings.weight", "token_embd.weight", "token_embd", "token_embeddings.weight"]


def dtype_name(raw: int) -> str:
    return DTYPE_NAMES.get(raw, f"Unknown({raw})")


class _Reader:
    def __init__(self, data: bytes):
        self.b, self.p = data, 0

    def take(self, n: int) -> bytes:
        if n < 0 or self.p + n > len(self.b):
            raise GgufError("failed to fill whole buffer")      # std::io::Read::read_exact
        out = self.b[self.p:self.p + n]
        self.p += n
        return out

    def fmt(self, f: str):
        return struct.unpack(f, self.take(struct.calcsize(f)))[0]

    def string(self) -> str:                                    # src/gguf.rs:368-375
        n = self.fmt("<Q")
        raw = self.take(n)
        try:
            return raw.decode("utf-8")
        except UnicodeDecodeError:
            raise GgufError("GGUF string is not valid UTF-8")

    def scalar(self, vt: int):                                  # src/gguf.rs:377-421
        if vt in _SCALAR_FMT:
            return (vt, self.fmt(_SCALAR_FMT[vt]))
        if vt == BOOL:
            return (vt, self.take(1)[0] != 0)
        if vt == STR:
            return (vt, self.string())
        raise GgufError("read_scalar called with ARRAY type")


def _align(offset: int, alignment: int) -> int:                 # src/gguf.rs:293-301
    rem = offset % alignment
    return offset if rem == 0 else offset + (alignment - rem)


def _payload_end(t: dict):                                      # src/gguf.rs:303-329
    lay = DTYPE_LAYOUT.get(t["dtype"])
    if lay is None:
        return None
    elems = 1
    for d in t["shape"]:
        elems *= d
        if elems >= 1 << 64:
            return None
    blocks = -(-elems // lay[0])
    end = t["offset"] + blocks * lay[1]
    return end if end < (1 << 64) and blocks * lay[1] < (1 << 64) else None


def load_gguf(data: bytes) -> dict:
    """src/gguf.rs:172-289.  Returns {version, metadata {key: (type, value) | ('array', elem_type, [values])},
    tensors [{name, dtype, dtype_raw, shape, offset}], data_offset}."""
    r = _Reader(data)
    if r.take(4) != b"GGUF":
        raise GgufError("Not a GGUF file (magic != GGUF)")
    version = r.fmt("<I")
    n_tensors, n_kv = r.fmt("<Q"), r.fmt("<Q")
    metadata = {}
    for _ in range(n_kv):
        key = r.string()
        vt = r.fmt("<I")
        if vt > F64:
            raise GgufError(f"unknown GGUF value type: {vt}")
        if vt == ARRAY:
            et = r.fmt("<I")
            if et > F64:
                raise GgufError(f"unknown GGUF array element type: {et}")
            n = r.fmt("<Q")
            metadata[key] = ("array", et, [r.scalar(et)[1] for _ in range(n)])
        else:
            metadata[key] = r.scalar(vt)
    tensors = []
    for _ in range(n_tensors):
        name = r.string()
        nd = r.fmt("<I")
        shape = [r.fmt("<Q") for _ in range(nd)]
        raw = r.fmt("<I")
        off = r.fmt("<Q")
        tensors.append(dict(name=name, dtype=dtype_name(raw), dtype_raw=raw, shape=shape, offset=off))
    info_end, file_len = r.p, len(data)
    ends = [e for e in (_payload_end(t) for t in tensors) if e is not None]
    max_end = max(ends) if ends else 0
    al = metadata.get("general.alignment")
    if al is not None:
        if al[0] in (U32, U64, I32, I64) and al[1] > 0:
            data_offset = _align(info_end, al[1])
        else:
            raise GgufError("general.alignment must be a positive integer when present")
    elif tensors:
        aligned = _align(info_end, 32)
        data_offset = aligned if aligned + max_end <= file_len else info_end
    else:
        data_offset = info_end
    return dict(version=version, metadata=metadata, tensors=tensors, data_offset=data_offset)


# ---- metadata accessors (src/infer/meta.rs:5-21, 139-154) ------------------------------------------------
def get_u32(meta: dict, key: str):
    v = meta.get(key)
    if v is None or v[0] not in (U32, I32, U64, I64):
        return None
    return v[1] if 0 <= v[1] < (1 << 32) else None


def get_u32_any(meta, keys):
    for k in keys:
        v = get_u32(meta, k)
        if v is not None:
            return v
    return None


def get_f32_any(meta, keys):
    for k in keys:
        v = meta.get(k)
        if v is not None and v[0] == F32:
            return np.float32(v[1])
    return None


def _find(tensors, name):
    return next((t for t in tensors if t["name"] == name), None)


def model_config_from_metadata(meta: dict, tensors: list) -> dict:
    """src/infer/types.rs:114-242 with the derive_* helpers of src/infer/meta.rs:23-137."""
    a = meta.get("general.architecture")
    if a is None or a[0] != STR:
        raise GgufError("missing general.architecture")
    arch = a[1]

    def need(suffix, label):
        v = get_u32_any(meta, [f"{arch}.{suffix}", f"llama.{suffix}"])
        if v is None:
            raise GgufError(f"missing architecture {label}")
        return v

    d = need("embedding_length", "embedding_length")
    heads = need("attention.head_count", "attention.head_count")
    blocks = need("block_count", "block_count")
    ctx_len = need("context_length", "context_length")
    # feed_forward_length (meta.rs:99-137)
    ff = get_u32_any(meta, [f"{arch}.feed_forward_length", "llama.feed_forward_length"])
    if ff is not None:
        if ff == 0:
            raise GgufError("feed_forward_length must be > 0")
    else:
        for name in ["layers.0.feed_forward.w1.weight", "layers.0.feed_forward.w3.weight", "blk.0.ffn_gate.weight",
                     "blk.0.ffn_up.weight", "layers.0.ffn_gate.weight", "layers.0.ffn_up.weight"]:
            t = _find(tensors, name)
            if t is not None:
                if len(t["shape"]) != 2:
                    raise GgufError(f"feed-forward tensor {name} must be rank-2")
                k, n = t["shape"][0] & 0xffffffff, t["shape"][1] & 0xffffffff
                if k == d and n > 0:
                    ff = n
                    break
        if ff is None:
            raise GgufError("feed_forward_length missing; add architecture feed_forward_length or a feed-forward weight tensor")
    hd = get_u32_any(meta, [f"{arch}.attention.key_length", "llama.attention.key_length"])
    if hd is None:
        if heads == 0:
            raise GgufError("attention_head_count must be > 0")     # the reference divides by zero here
        hd = d // heads
    # kv heads (meta.rs:23-58)
    kvh = get_u32_any(meta, [f"{arch}.attention.head_count_kv", "llama.attention.head_count_kv"])
    if kvh is None:
        for name in ["layers.0.attention.wk.weight", "blk.0.attn_k.weight", "layers.0.attention.wv.weight", "blk.0.attn_v.weight"]:
            t = _find(tensors, name)
            if t is not None:
                if len(t["shape"]) != 2:
                    raise GgufError(f"attention tensor {name} must be rank-2")
                k, n = t["shape"][0] & 0xffffffff, t["shape"][1] & 0xffffffff
                if k == d and n > 0 and hd > 0 and n % hd == 0:
                    kvh = n // hd
                    break
        if kvh is None:
            kvh = heads
    eps = get_f32_any(meta, [f"{arch}.attention.layer_norm_rms_epsilon", f"{arch}.layer_norm_epsilon", "llama.layer_norm_epsilon"])
    eps = np.float32(1e-5) if eps is None else eps
    base = get_f32_any(meta, [f"{arch}.rope.freq_base", "llama.rope.freq_base"])
    base = np.float32(10000.0) if base is None else base
    scale = get_f32_any(meta, [f"{arch}.rope.freq_scale", "llama.rope.freq_scale"])
    scale = np.float32(1.0) if scale is None else scale
    # vocab (meta.rs:60-97)
    vocab = get_u32_any(meta, [f"{arch}.vocab_size", "llama.vocab_size"])
    if vocab is not None:
        if vocab == 0:
            raise GgufError("vocab_size must be > 0")
    else:
        for name in EMBEDDING_NAMES:
            t = _find(tensors, name)
            if t is not None:
                if len(t["shape"]) != 2:
                    raise GgufError(f"embedding tensor {name} must be rank-2")
                r0, r1 = t["shape"][0] & 0xffffffff, t["shape"][1] & 0xffffffff
                if r0 == d and r1 > 0:
                    vocab = r1
                    break
                if r1 == d and r0 > 0:
                    vocab = r0
                    break
        if vocab is None:
            raise GgufError("vocab_size missing; add architecture vocab_size or embeddings tensor")
    cfg = dict(architecture=arch, block_count=blocks, context_length=ctx_len, embedding_length=d, feed_forward_length=ff,
               attention_head_count=heads, attention_head_count_kv=kvh, attention_key_length=hd,
               layer_norm_epsilon=float(eps), rope_freq_base=float(base), rope_freq_scale=float(scale), vocab_size=vocab,
               rope_layout=1 if arch.startswith("qwen") else 0)       # types.rs:34-40
    # validate (types.rs:181-241)
    for key in ("embedding_length", "attention_head_count", "block_count", "context_length", "feed_forward_length",
                "vocab_size", "attention_head_count_kv", "attention_key_length"):
        if cfg[key] == 0:
            raise GgufError(f"{key} must be > 0")
    if d != (heads * hd) & 0xffffffff:
        raise GgufError(f"embedding_length {d} must equal attention_head_count {heads} * attention_key_length {hd}")
    if d % heads:
        raise GgufError(f"embedding_length {d} not divisible by attention_head_count {heads}")
    if heads % kvh:
        raise GgufError(f"attention_head_count {heads} not divisible by attention_head_count_kv {kvh}")
    if not np.isfinite(base) or base <= 0:
        raise GgufError("rope_freq_base must be finite and > 0")
    if not np.isfinite(scale) or scale <= 0:
        raise GgufError("rope_freq_scale must be finite and > 0")
    return cfg


def build_tensor_views(tensors: list, weights_len: int) -> dict:
    """src/infer/load.rs:41-63 (blob bounds, first) then src/infer/tensor_views.rs:8-117."""
    for t in tensors:
        lay = DTYPE_LAYOUT.get(t["dtype"])
        if lay is not None:
            n = 1
            for dim in t["shape"]:
                n = (n * dim) & ((1 << 64) - 1)
            need = -(-n // lay[0]) * lay[1]
            end = min(t["offset"] + need, (1 << 64) - 1)
            if end > weights_len:
                raise GgufError(f"tensor '{t['name']}' overflows weights blob: [{t['offset']}..{end}) > {weights_len}")
    views = {}
    for t in tensors:
        name = t["name"]
        if not t["shape"]:
            raise GgufError(f"tensor '{name}' has empty shape")
        for i, dim in enumerate(t["shape"]):
            if dim == 0:
                raise GgufError(f"tensor '{name}' has zero in dimension {i}")
        align = {"F16": 2, "F32": 4}.get(t["dtype"], 1)
        if align > 1 and t["offset"] % align:
            raise GgufError(f"tensor '{name}' offset {t['offset']} misaligned for {t['dtype']} (align {align})")
        lay = DTYPE_LAYOUT.get(t["dtype"])
        if lay is None:
            raise GgufError(f"tensor '{name}' unsupported dtype: {t['dtype']}")
        n = 1
        for dim in t["shape"]:
            n *= dim
        need = -(-n // lay[0]) * lay[1]
        if t["offset"] + need > weights_len:
            raise GgufError(f"tensor '{name}' overflows weights blob or starts beyond end (off={t['offset']}, nbytes={need}, total={weights_len})")
        strides, s = [], 1
        for dim in reversed(t["shape"]):
            strides.append(s)
            s *= dim
        views[name] = dict(dtype=t["dtype"], shape=list(t["shape"]), strides=strides[::-1], byte_offset=t["offset"], nbytes=need)
    return views


# ---- tensor-name mapping (src/infer/mapping.rs) ----------------------------------------------------------
def _first(views, names):
    for n in names:
        if n in views:
            return n
    return None


def _require(views, names):
    n = _first(views, names)
    if n is None:
        raise GgufError("missing required tensor; tried: " + ", ".join(names))
    return n


def _norm_check(label, v, dim):                                 # mapping.rs:76-91
    if v["dtype"] not in ("F16", "F32"):
        raise GgufError(f"{label} expected F16 or F32, got {v['dtype']}")
    if len(v["shape"]) != 1 or v["shape"][0] != dim:
        raise GgufError(f"{label} shape invalid: expected [{dim}], got {v['shape']}")


def map_standard_layer(views: dict, cfg: dict, layer: int) -> dict:
    """src/infer/mapping.rs:95-353.  Returns the chosen tensor name per role (None for absent optional ones)
    plus d_model and hidden_dim."""
    tok_name = _require(views, EMBEDDING_NAMES)
    tok = views[tok_name]
    if tok["dtype"] not in ("F16", "Q8_0"):
        raise GgufError(f"tok_embeddings.weight expected F16 or Q8_0 [*, *], got {tok['dtype']}")
    if len(tok["shape"]) != 2:
        raise GgufError(f"embeddings shape invalid: expected rank-2, got {tok['shape']}")
    r0, r1 = tok["shape"]
    d = cfg["embedding_length"]
    if r1 == d:
        vocab_dim = r0
    elif r0 == d:
        vocab_dim = r1
    else:
        raise GgufError(f"embeddings dims {tok['shape']} do not contain d_model {d}")
    if cfg["vocab_size"] != vocab_dim:
        raise GgufError(f"vocab_size meta {cfg['vocab_size']} != embeddings vocab dim {vocab_dim} (shape={tok['shape']})")
    if layer >= cfg["block_count"]:
        raise GgufError(f"layer {layer} out of range (block_count={cfg['block_count']})")
    L = layer
    cand = dict(
        wq=[f"layers.{L}.attention.wq.weight", f"blk.{L}.attn_q.weight"],
        wk=[f"layers.{L}.attention.wk.weight", f"blk.{L}.attn_k.weight"],
        wv=[f"layers.{L}.attention.wv.weight", f"blk.{L}.attn_v.weight"],
        bq=[f"layers.{L}.attention.wq.bias", f"blk.{L}.attn_q.bias"],
        bk=[f"layers.{L}.attention.wk.bias", f"blk.{L}.attn_k.bias"],
        bv=[f"layers.{L}.attention.wv.bias", f"blk.{L}.attn_v.bias"],
        wo=[f"layers.{L}.attention.wo.weight", f"blk.{L}.attn_output.weight"],
        w_gate=[f"layers.{L}.feed_forward.w3.weight", f"blk.{L}.ffn_gate.weight"],
        w_up=[f"layers.{L}.feed_forward.w1.weight", f"blk.{L}.ffn_up.weight"],
        w_down=[f"layers.{L}.feed_forward.w2.weight", f"blk.{L}.ffn_down.weight"],
        attn_norm=[f"layers.{L}.attention_norm.weight", f"layers.{L}.attn_norm.weight", f"blk.{L}.attn_norm.weight"],
        ffn_norm=[f"layers.{L}.ffn_norm.weight", f"layers.{L}.feed_forward_norm.weight", f"blk.{L}.ffn_norm.weight"])
    out = {}
    for role in ("wq", "wk", "wv"):
        out[role] = _require(views, cand[role])
    for role in ("bq", "bk", "bv"):
        out[role] = _first(views, cand[role])
    for role in ("wo", "w_gate", "w_up", "w_down"):
        out[role] = _require(views, cand[role])
    for role in ("attn_norm", "ffn_norm"):
        out[role] = _first(views, cand[role])
    for role in ("wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down"):
        if views[out[role]]["dtype"] not in ("F16", "Q5_1"):
            raise GgufError(f"tensor {role} expected F16 or Q5_1, got {views[out[role]]['dtype']}")

    def dims(role):
        s = views[out[role]]["shape"]
        return (s[0] if len(s) > 0 else 0), (s[1] if len(s) > 1 else 0)

    for role in ("wq", "wk", "wv", "wo"):
        k, n = dims(role)
        if k != d or n == 0:
            raise GgufError(f"{role} shape invalid: expected [d_model, N], got {views[out[role]]['shape']}")
    hd, nh, nkv = cfg["attention_key_length"], cfg["attention_head_count"], cfg["attention_head_count_kv"]
    for role, exp in (("wq", nh * hd), ("wk", nkv * hd), ("wv", nkv * hd), ("wo", d)):
        if dims(role)[1] != exp:
            raise GgufError(f"{role} second dim {dims(role)[1]} != expected {exp}")
    for role, exp in (("bq", nh * hd), ("bk", nkv * hd), ("bv", nkv * hd)):
        if out[role] is not None:
            v = views[out[role]]
            if v["dtype"] != "F32":
                raise GgufError(f"{role} expected F32 bias, got {v['dtype']}")
            if len(v["shape"]) != 1 or v["shape"][0] != exp:
                raise GgufError(f"{role} shape invalid: expected [{exp}], got {v['shape']}")
    for role in ("w_gate", "w_up"):
        k, h = dims(role)
        if k != d or h == 0:
            raise GgufError(f"{role} shape invalid: expected [d_model, H], got {views[out[role]]['shape']}")
    hidden = dims("w_up")[1]
    if dims("w_down") != (hidden, d):
        raise GgufError(f"w_down shape invalid: expected [hidden_dim, d_model]=[{hidden}, {d}], got {views[out['w_down']]['shape']}")
    if cfg["feed_forward_length"] != hidden:
        raise GgufError(f"model_config.feed_forward_length {cfg['feed_forward_length']} != inferred hidden_dim {hidden}")
    if out["attn_norm"] is not None:
        _norm_check("attention norm", views[out["attn_norm"]], d)
    if out["ffn_norm"] is not None:
        _norm_check("ffn norm", views[out["ffn_norm"]], d)
    out.update(tok_embeddings=tok_name, d_model=d, hidden_dim=hidden)
    return out


def map_lm_head(views: dict, cfg: dict) -> dict:
    """src/infer/mapping.rs:360-437: a dedicated output tensor first, else F16 embeddings already laid out
    as [d_model, vocab]."""
    name = _first(views, ["output.weight", "lm_head.weight", "output"])
    if name is not None:
        t = views[name]
        if t["dtype"] != "F16":
            raise GgufError(f"lm_head expected F16, got {t['dtype']}")
        if len(t["shape"]) != 2:
            raise GgufError(f"lm_head shape invalid: expected [d_model, vocab], got {t['shape']}")
        if t["shape"][0] == 0 or t["shape"][1] == 0:
            raise GgufError(f"lm_head dims invalid: non-zero [d_model, vocab] required: {t['shape']}")
        return dict(name=name, d_model=t["shape"][0], vocab=t["shape"][1], tied=False)
    name = _first(views, EMBEDDING_NAMES)
    if name is not None:
        t = views[name]
        if t["dtype"] != "F16":
            raise GgufError(f"tied lm_head requires F16 embeddings when output head is absent; tensor {name} has {t['dtype']}")
        if len(t["shape"]) != 2:
            raise GgufError(f"tied lm_head embedding shape invalid: expected [d_model, vocab], got {t['shape']}")
        d, v = cfg["embedding_length"], cfg["vocab_size"]
        if t["shape"][0] != d or t["shape"][1] != v:
            raise GgufError(f"tied lm_head embedding layout unsupported: expected [d_model, vocab]=[{d}, {v}], got {t['shape']}")
        return dict(name=name, d_model=d, vocab=v, tied=True)
    raise GgufError("output projection tensor not found; expected one of output.weight, lm_head.weight, output or tied F16 "
                    "embeddings in [d_model, vocab] layout")


def map_output_norm(views: dict, cfg: dict):
    """src/infer/mapping.rs:439-459."""
    name = _first(views, ["output_norm.weight", "norm.weight", "model.norm.weight"])
    if name is None:
        return None
    _norm_check("output norm", views[name], cfg["embedding_length"])
    return name


def validate_standard_layers(views: dict, cfg: dict):
    """src/infer/mapping.rs:461-493."""
    if cfg["block_count"] == 0:
        raise GgufError("model_config.block_count must be > 0")
    d = h = None
    for layer in range(cfg["block_count"]):
        w = map_standard_layer(views, cfg, layer)
        if d is not None and d != w["d_model"]:
            raise GgufError(f"layer {layer} d_model mismatch: expected {d}, got {w['d_model']}")
        if h is not None and h != w["hidden_dim"]:
            raise GgufError(f"layer {layer} hidden_dim mismatch: expected {h}, got {w['hidden_dim']}")
        d, h = w["d_model"], w["hidden_dim"]
    return d, h


def token_embedding_f32(weights: bytes, views: dict, cfg: dict, token_id: int) -> np.ndarray:
    """src/infer/embeddings.rs:14-143 for F16 and Q8_0 tables.  In either orientation the token's d_model
    values are contiguous (dimension 0 of a GGUF shape is the fastest one), so both branches of the
    reference read `token_id * row_bytes`."""
    name = _require(views, EMBEDDING_NAMES)
    tok = views[name]
    if len(tok["shape"]) != 2:
        raise GgufError("embeddings must be [vocab, d_model]")
    r0, r1 = tok["shape"]
    d, vsz = cfg["embedding_length"], cfg["vocab_size"]
    rows_are_vocab = True if vsz == r0 else False if vsz == r1 else True if r1 == d else False if r0 == d else (r1 == d)
    vocab = r0 if rows_are_vocab else r1
    if token_id >= vocab:
        raise GgufError(f"token_id {token_id} out of range for vocab size {vocab}")
    base = tok["byte_offset"]
    if tok["dtype"] == "F16":
        off = base + token_id * d * 2
        return np.frombuffer(weights, dtype=np.float16, count=d, offset=off).astype(np.float32)
    if tok["dtype"] == "Q8_0":
        blocks = -(-d // 32)
        off = base + token_id * blocks * 34
        out = np.zeros(d, dtype=np.float32)
        for b in range(blocks):
            o = off + b * 34
            scale = np.frombuffer(weights, dtype=np.float16, count=1, offset=o).astype(np.float32)[0]
            q = np.frombuffer(weights, dtype=np.int8, count=32, offset=o + 2).astype(np.float32)
            n = min(32, d - b * 32)
            out[b * 32:b * 32 + n] = scale * q[:n]
        return out
    raise GgufError(f"unsupported embedding dtype: {tok['dtype']}")
