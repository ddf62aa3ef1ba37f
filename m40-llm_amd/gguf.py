"""ctypes view of the host layer's GGUF ingestion (m40host_gguf_* in include/m40llm_host.h): the header of a
file as a dictionary, and a file whose tensors are resident on the device with a decoder reading them in place.
Mirrors the reference's load_gguf + LoadedModel::from_gguf (src/gguf.rs:172, src/infer/load.rs:11)."""
from __future__ import annotations

import ctypes as C
import json

import numpy as np

from . import Context, host
from .synthetic import DeviceModel, HostKvConfig


class GgufError(RuntimeError):
    pass


def _describe(H, handle) -> dict:
    n = H.m40host_gguf_describe_json(handle, None, 0)
    buf = C.create_string_buffer(n)
    H.m40host_gguf_describe_json(handle, buf, n)
    return json.loads(buf.value.decode("utf-8"))


def describe_file(path: str) -> dict:
    """Parse a file's header (no device) and return everything the host layer derives from it."""
    H = host()
    h = H.m40host_gguf_open(path.encode())
    if not h:
        raise GgufError(H.m40host_last_error().decode())
    try:
        return _describe(H, h)
    finally:
        H.m40host_gguf_close(h)


def describe_bytes(data: bytes) -> dict:
    H = host()
    h = H.m40host_gguf_parse(data, len(data))
    if not h:
        raise GgufError(H.m40host_last_error().decode())
    try:
        return _describe(H, h)
    finally:
        H.m40host_gguf_close(h)


def embedding_row(data: bytes, token_id: int):
    """(byte offset in the data section, row bytes, ggml dtype code) of one token's embedding."""
    H = host()
    h = H.m40host_gguf_parse(data, len(data))
    if not h:
        raise GgufError(H.m40host_last_error().decode())
    try:
        off, nb, dt = C.c_uint64(), C.c_uint64(), C.c_uint32()
        if H.m40host_gguf_embedding_row(h, token_id, C.byref(off), C.byref(nb), C.byref(dt)) != 0:
            raise GgufError(H.m40host_last_error().decode())
        return off.value, nb.value, dt.value
    finally:
        H.m40host_gguf_close(h)


class GgufModel(DeviceModel):
    """A decoder whose weights are the tensors of a loaded file (no copies, no repacking)."""

    def __init__(self, weights: "GgufWeights", handle, cfg: dict, max_seq_len: int, max_sequences: int):
        self.ctx, self.cfg, self.H, self.h = weights.ctx, cfg, weights.H, handle
        self.weights = weights          # keeps the device allocation alive
        self.bufs = []
        self.weight_bytes = weights.weights_len
        self.max_seq_len, self.max_sequences = max_seq_len, max_sequences


class GgufWeights:
    def __init__(self, ctx: Context, path: str):
        self.ctx, self.H, self.path = ctx, host(), path
        self.h = self.H.m40host_gguf_load(ctx.h, path.encode())
        if not self.h:
            raise GgufError(self.H.m40host_last_error().decode())
        self.weights_len = self.H.m40host_gguf_weights_len(self.h)
        self.base = self.H.m40host_gguf_weights_base(self.h)
        self.info = describe_file(path)

    def close(self):
        if getattr(self, "h", None):
            self.H.m40host_gguf_weights_free(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def tensor_ptr(self, name: str) -> int:
        p = self.H.m40host_gguf_tensor_ptr(self.h, name.encode())
        if not p:
            raise GgufError(self.H.m40host_last_error().decode())
        return p

    def read_tensor_bytes(self, name: str) -> bytes:
        v = self.info["views"][name]
        out = np.empty(v["nbytes"], dtype=np.uint8)
        rc = self.ctx.lib.m40llm_memcpy_d2h(self.ctx.h, out.ctypes.data_as(C.c_void_p), self.tensor_ptr(name), v["nbytes"])
        if rc != 0:
            raise GgufError(f"m40llm_memcpy_d2h -> {rc}")
        return out.tobytes()

    def token_embedding(self, token_id: int) -> np.ndarray:
        d = self.info["config"]["embedding_length"]
        buf = self.ctx.alloc(d * 4)
        if self.H.m40host_gguf_load_token_embedding_f32(self.h, token_id, buf.ptr) != 0:
            raise GgufError(self.H.m40host_last_error().decode())
        return buf.download(np.float32, (d,))

    def model(self, max_seq_len: int = 0, max_sequences: int = 1, kv_cfg: dict | None = None) -> GgufModel:
        kc = None
        if kv_cfg is not None:
            kc = HostKvConfig(kv_cfg.get("mode", 2), kv_cfg["recent_window"], kv_cfg["block_size"], kv_cfg["top_blocks"], 0, 0,
                              kv_cfg.get("exact_old_backing", 2), kv_cfg.get("exact_old_attention", 2))
        h = self.H.m40host_model_from_gguf(self.h, max_seq_len, max_sequences, C.byref(kc) if kc is not None else None)
        if not h:
            raise GgufError(self.H.m40host_last_error().decode())
        c = self.info["config"]
        cfg = dict(n_layers=c["block_count"], d_model=c["embedding_length"], q_heads=c["attention_head_count"],
                   kv_heads=c["attention_head_count_kv"], head_dim=c["attention_key_length"], ffn=c["feed_forward_length"],
                   vocab=c["vocab_size"], rms_eps=c["layer_norm_epsilon"], rope_base=c["rope_freq_base"],
                   rope_scale=c["rope_freq_scale"], rope_layout=c["rope_layout"],
                   qkv_bias=self.info["layers"][0].get("bq") is not None)
        return GgufModel(self, h, cfg, max_seq_len or c["context_length"], max_sequences)


def write_model_file(path: str, cfg: dict, W: dict, arch: str = "llama", alignment: int = 32) -> int:
    """Stream a synthetic decoder (the weight dictionary of synthetic.make_weights) to `path` as a GGUF v3 file with
    llama.cpp's tensor names (blk.N.*, token_embd, output_norm, output); shapes are written fastest dimension first
    ([K, N] for a projection with N output columns).  Returns the file size.  Used by the load benchmark; nothing is
    converted: the f16 arrays go to the file as they are."""
    import struct

    def s(x: str) -> bytes:
        raw = x.encode()
        return struct.pack("<Q", len(raw)) + raw

    kvs = [s("general.architecture") + struct.pack("<I", 8) + s(arch)]
    for key, val in (("block_count", cfg["n_layers"]), ("embedding_length", cfg["d_model"]), ("attention.head_count", cfg["q_heads"]),
                     ("attention.head_count_kv", cfg["kv_heads"]), ("context_length", cfg.get("context_length", 2048)),
                     ("feed_forward_length", cfg["ffn"]), ("vocab_size", cfg["vocab"])):
        kvs.append(s(f"{arch}.{key}") + struct.pack("<II", 4, val))
    for key, val in (("attention.layer_norm_rms_epsilon", cfg["rms_eps"]), ("rope.freq_base", cfg["rope_base"])):
        kvs.append(s(f"{arch}.{key}") + struct.pack("<If", 6, val))
    tensors = [("token_embd.weight", W["tok_emb"], 1)]
    for l in range(cfg["n_layers"]):
        tensors.append((f"blk.{l}.attn_norm.weight", W["attn_norm"][l], 0))
        for role, name in (("wq", "attn_q"), ("wk", "attn_k"), ("wv", "attn_v")):
            tensors.append((f"blk.{l}.{name}.weight", W[role][l], 1))
        if cfg.get("qkv_bias"):
            for role, name in (("bq", "attn_q"), ("bk", "attn_k"), ("bv", "attn_v")):
                tensors.append((f"blk.{l}.{name}.bias", W[role][l], 0))
        tensors.append((f"blk.{l}.attn_output.weight", W["wo"][l], 1))
        tensors.append((f"blk.{l}.ffn_norm.weight", W["ffn_norm"][l], 0))
        for role, name in (("wgate", "ffn_gate"), ("wup", "ffn_up"), ("wdown", "ffn_down")):
            tensors.append((f"blk.{l}.{name}.weight", W[role][l], 1))
    tensors.append(("output_norm.weight", W["out_norm"], 0))
    if W["lm_head"] is not W["tok_emb"]:
        tensors.append(("output.weight", W["lm_head"], 1))
    head = b"GGUF" + struct.pack("<IQQ", 3, len(tensors), len(kvs)) + b"".join(kvs)
    offsets, at = [], 0
    for name, a, dt in tensors:
        at += -at % alignment
        offsets.append(at)
        at += a.nbytes
        shape = list(a.shape)[::-1]
        head += s(name) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", d) for d in shape) + struct.pack("<IQ", dt, offsets[-1])
    with open(path, "wb") as f:
        f.write(head)
        f.write(b"\0" * (-len(head) % alignment))
        pos = 0
        for (name, a, dt), off in zip(tensors, offsets):
            f.write(b"\0" * (off - pos))
            f.write(np.ascontiguousarray(a).data)
            pos = off + a.nbytes
        return f.tell()
