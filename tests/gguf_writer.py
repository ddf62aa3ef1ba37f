"""Writer of small GGUF files for the ingestion tests.  Independent of the parsers under test: it follows the
published container layout (magic, u32 version, u64 tensor count, u64 metadata count, metadata pairs, tensor
descriptors, data section) the same way the reference's tests write their files
(tests/gguf_device_views_offsets.rs:8-43, tests/gguf_metadata_config.rs:8-26)."""
from __future__ import annotations

import struct

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STR, ARRAY, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q", I64: "<q", F64: "<d"}
F32_T, F16_T, Q4_0_T, Q5_1_T, Q8_0_T = 0, 1, 2, 7, 8


def _string(s) -> bytes:
    raw = s if isinstance(s, bytes) else s.encode("utf-8")
    return struct.pack("<Q", len(raw)) + raw


def _scalar(vt: int, v) -> bytes:
    return _string(v) if vt == STR else struct.pack(_FMT[vt], v)


class GgufWriter:
    def __init__(self, version: int = 3):
        self.version = version
        self.kvs: list[bytes] = []
        self.tensors: list[tuple] = []      # (name, shape, dtype_raw, offset or None, payload bytes or None)

    def kv(self, key: str, vt: int, value):
        self.kvs.append(_string(key) + struct.pack("<I", vt) + _scalar(vt, value))
        return self

    def kv_array(self, key: str, elem_type: int, values):
        body = b"".join(_scalar(elem_type, v) for v in values)
        self.kvs.append(_string(key) + struct.pack("<II", ARRAY, elem_type) + struct.pack("<Q", len(values)) + body)
        return self

    def raw_kv(self, blob: bytes):
        self.kvs.append(blob)
        return self

    def tensor(self, name: str, shape, dtype_raw: int, offset=None, payload: bytes | None = None):
        self.tensors.append((name, list(shape), dtype_raw, offset, payload))
        return self

    def header(self, offsets) -> bytes:
        out = b"GGUF" + struct.pack("<IQQ", self.version, len(self.tensors), len(self.kvs)) + b"".join(self.kvs)
        for (name, shape, dt, _, _), off in zip(self.tensors, offsets):
            out += _string(name) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", d) for d in shape)
            out += struct.pack("<IQ", dt, off)
        return out

    def build_raw(self, data: bytes, pad_to: int | None = None) -> bytes:
        """Explicit offsets and an explicit data region, as the reference's tests write them (no padding unless
        pad_to is given)."""
        head = self.header([t[3] or 0 for t in self.tensors])
        if pad_to:
            head += b"\0" * (-len(head) % pad_to)
        return head + data

    def build(self, alignment: int = 32, write_alignment_key: bool = False) -> bytes:
        """Payloads laid out back to back, each aligned, data section aligned: what real converters write."""
        if write_alignment_key:
            self.kv("general.alignment", U32, alignment)
        offsets, at = [], 0
        for t in self.tensors:
            at += -at % alignment
            offsets.append(at)
            at += len(t[4])
        head = self.header(offsets)
        head += b"\0" * (-len(head) % alignment)
        data = bytearray(at)
        for t, off in zip(self.tensors, offsets):
            data[off:off + len(t[4])] = t[4]
        return head + bytes(data)


def llama_metadata(w: GgufWriter, arch="llama", **kv):
    """The seven keys of the reference tests' minimal metadata (tests/gguf_device_views_offsets.rs:28-36), with
    overrides; a value of None leaves the key out."""
    base = dict(embedding_length=4, head_count=1, block_count=1, context_length=16, feed_forward_length=8, vocab_size=32)
    base.update(kv)
    w.kv("general.architecture", STR, arch)
    names = dict(embedding_length="embedding_length", head_count="attention.head_count", block_count="block_count",
                 context_length="context_length", feed_forward_length="feed_forward_length", vocab_size="vocab_size",
                 head_count_kv="attention.head_count_kv", key_length="attention.key_length")
    for k, v in base.items():
        if v is None:
            continue
        if k in names:
            w.kv(f"{arch}.{names[k]}", U32, v)
        else:                                   # full key with (type, value)
            w.kv(k, v[0], v[1])
    return w


def q80_blocks(values: np.ndarray) -> bytes:
    """Quantise rows of f32 (length a multiple of 32) to 34-byte q8_0 blocks: f16 scale d = max|x| / 127, then
    round(x / d)."""
    v = np.asarray(values, dtype=np.float32).reshape(-1, 32)
    d = (np.abs(v).max(axis=1) / np.float32(127.0)).astype(np.float16)
    df = d.astype(np.float32)
    q = np.where(df[:, None] > 0, np.rint(v / np.where(df == 0, 1, df)[:, None]), 0).clip(-127, 127).astype(np.int8)
    out = bytearray()
    for i in range(v.shape[0]):
        out += d[i].tobytes() + q[i].tobytes()
    return bytes(out)


def model_file(cfg: dict, W: dict, arch: str = "llama", naming: str = "blk", tied: bool = False,
               norm_f16: bool = False, drop: tuple = (), alignment: int = 32) -> bytes:
    """A whole decoder as a GGUF file from the weight dictionary of m40-llm_amd/synthetic.make_weights (weights as
    uint16 views of f16 [N][K]); shapes are written GGUF-style, fastest dimension first: [K, N]."""
    w = GgufWriter()
    w.kv("general.architecture", STR, arch)
    w.kv(f"{arch}.block_count", U32, cfg["n_layers"])
    w.kv(f"{arch}.embedding_length", U32, cfg["d_model"])
    w.kv(f"{arch}.attention.head_count", U32, cfg["q_heads"])
    w.kv(f"{arch}.attention.head_count_kv", U32, cfg["kv_heads"])
    w.kv(f"{arch}.context_length", U32, cfg.get("context_length", 64))
    w.kv(f"{arch}.feed_forward_length", U32, cfg["ffn"])
    w.kv(f"{arch}.attention.layer_norm_rms_epsilon", F32, cfg["rms_eps"])
    w.kv(f"{arch}.rope.freq_base", F32, cfg["rope_base"])
    w.kv(f"{arch}.vocab_size", U32, cfg["vocab"])
    w.kv_array("tokenizer.ggml.tokens", STR, [f"<t{i}>" for i in range(40)])
    w.kv_array("tokenizer.ggml.scores", F32, [float(-i) for i in range(40)])

    def f16(name, a):          # a: uint16 [N][K]
        if name not in drop:
            w.tensor(name, [a.shape[1], a.shape[0]], F16_T, payload=np.ascontiguousarray(a).tobytes())

    def norm(name, a):
        if name in drop:
            return
        if norm_f16:
            w.tensor(name, [a.shape[0]], F16_T, payload=a.astype(np.float16).tobytes())
        else:
            w.tensor(name, [a.shape[0]], F32_T, payload=a.astype(np.float32).tobytes())

    f16("token_embd.weight" if naming == "blk" else "tok_embeddings.weight", W["tok_emb"])
    for l in range(cfg["n_layers"]):
        if naming == "blk":
            n = dict(wq=f"blk.{l}.attn_q.weight", wk=f"blk.{l}.attn_k.weight", wv=f"blk.{l}.attn_v.weight",
                     wo=f"blk.{l}.attn_output.weight", wgate=f"blk.{l}.ffn_gate.weight", wup=f"blk.{l}.ffn_up.weight",
                     wdown=f"blk.{l}.ffn_down.weight", attn_norm=f"blk.{l}.attn_norm.weight", ffn_norm=f"blk.{l}.ffn_norm.weight",
                     bq=f"blk.{l}.attn_q.bias", bk=f"blk.{l}.attn_k.bias", bv=f"blk.{l}.attn_v.bias")
        else:
            n = dict(wq=f"layers.{l}.attention.wq.weight", wk=f"layers.{l}.attention.wk.weight",
                     wv=f"layers.{l}.attention.wv.weight", wo=f"layers.{l}.attention.wo.weight",
                     wgate=f"layers.{l}.feed_forward.w3.weight", wup=f"layers.{l}.feed_forward.w1.weight",
                     wdown=f"layers.{l}.feed_forward.w2.weight", attn_norm=f"layers.{l}.attention_norm.weight",
                     ffn_norm=f"layers.{l}.ffn_norm.weight", bq=f"layers.{l}.attention.wq.bias",
                     bk=f"layers.{l}.attention.wk.bias", bv=f"layers.{l}.attention.wv.bias")
        norm(n["attn_norm"], W["attn_norm"][l])
        for role in ("wq", "wk", "wv"):
            f16(n[role], W[role][l])
        if cfg.get("qkv_bias"):
            for role in ("bq", "bk", "bv"):
                w.tensor(n[role], [W[role][l].shape[0]], F32_T, payload=W[role][l].astype(np.float32).tobytes())
        f16(n["wo"], W["wo"][l])
        norm(n["ffn_norm"], W["ffn_norm"][l])
        for role in ("wgate", "wup", "wdown"):
            f16(n[role], W[role][l])
    norm("output_norm.weight", W["out_norm"])
    if not tied:
        f16("output.weight", W["lm_head"])
    return w.build(alignment=alignment, write_alignment_key=alignment != 32)
