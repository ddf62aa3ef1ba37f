"""GGUF ingestion on the GPU: the data section of a file lands on the device byte for byte, embedding rows come
out as the reference's host dequant computes them, and a decoder assembled from a file's tensors produces the
same token ids as the CPU oracle running on the same weights."""
import importlib
import os
import tempfile

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from gguf_writer import F16_T, F32_T, Q8_0_T, GgufWriter, llama_metadata, model_file  # noqa: E402
from gpu_common import close, m40  # noqa: E402
from test_gguf import reference_embedding_cases  # noqa: E402

gg = importlib.import_module("m40-llm_amd.gguf")
syn = importlib.import_module("m40-llm_amd.synthetic")


@pytest.fixture(scope="module")
def ctx():
    yield m40.Context(0)


@pytest.fixture()
def tmpfile():
    paths = []

    def make(data: bytes) -> str:
        fd, path = tempfile.mkstemp(suffix=".gguf")
        with os.fdopen(fd, "wb") as f:
            f.write(data)
        paths.append(path)
        return path
    yield make
    for p in paths:
        os.unlink(p)


def _oracle_model(orc, cfg, W, max_seq, max_sequences):
    m = orc.Model(dict(cfg, qkv_bias=bool(cfg.get("qkv_bias"))), W)
    m.alloc_kv(max_seq, max_sequences)
    return m


def test_embedding_rows_reference_cases(ctx, tmpfile):
    # tests/embedding_dequant_cuda.rs:85-226, bit-exact (f16 widening and d * q are exact operations)
    for label, data, token, want in reference_embedding_cases():
        w = gg.GgufWeights(ctx, tmpfile(data))
        got = w.token_embedding(token)
        assert np.array_equal(got, want), label
        with pytest.raises(gg.GgufError, match="out of range"):
            w.token_embedding(w.info["config"]["vocab_size"])
        w.close()


def test_data_section_is_resident_byte_for_byte_across_staging_buffers(ctx, tmpfile):
    # 150 MiB of random bytes in three tensors: many rounds through the two staging buffers, offsets that are not
    # multiples of the buffer size
    rng = np.random.default_rng(0)
    sizes = [(1 << 20) * 70 + 6, (1 << 20) * 3, (1 << 20) * 77 + 2]
    blobs = [rng.integers(0, 65536, size=n // 2, dtype=np.uint16) for n in sizes]
    w = llama_metadata(GgufWriter())
    for i, b in enumerate(blobs):
        w.tensor(f"t{i}", [b.size], F16_T, payload=b.tobytes())
    path = tmpfile(w.build())
    gw = gg.GgufWeights(ctx, path)
    assert gw.weights_len == os.path.getsize(path) - gw.info["data_offset"]
    for i, b in enumerate(blobs):
        assert gw.tensor_ptr(f"t{i}") == gw.base + gw.info["views"][f"t{i}"]["byte_offset"]
        assert gw.read_tensor_bytes(f"t{i}") == b.tobytes()
    with pytest.raises(gg.GgufError, match="no tensor named"):
        gw.tensor_ptr("missing")
    gw.close()


@pytest.mark.parametrize("arch,naming,bias,norm_f16,tied,hd", [
    ("qwen2", "blk", True, False, False, 128),
    ("llama", "layers", False, True, True, 64),
    ("llama", "blk", False, False, False, 16),
])
def test_decoder_from_file_matches_oracle_and_uploaded_arrays(ctx, orc, tmpfile, arch, naming, bias, norm_f16, tied, hd):
    layout = 1 if arch == "qwen2" else 0
    cfg = dict(n_layers=3, d_model=4 * hd, q_heads=4, kv_heads=2, head_dim=hd, ffn=6 * 64, vocab=500, rms_eps=1e-5,
               rope_base=1e6 if layout else 10000.0, rope_scale=1.0, rope_layout=layout, qkv_bias=bias, context_length=32)
    W = syn.make_weights(cfg, seed=4, std=0.08, emb_std=None if tied else 1.0, tie_embeddings=tied)
    for l in range(cfg["n_layers"]):
        g = (1 + 0.1 * np.random.default_rng(l).standard_normal(cfg["d_model"])).astype(np.float32)
        W["attn_norm"][l] = g.astype(np.float16).astype(np.float32) if norm_f16 else g
    gw = gg.GgufWeights(ctx, tmpfile(model_file(cfg, W, arch=arch, naming=naming, tied=tied, norm_f16=norm_f16)))
    c = gw.info["config"]
    assert (c["rope_layout"], c["attention_head_count_kv"], c["attention_key_length"], c["vocab_size"]) == (layout, 2, hd, 500)
    assert gw.info["lm_head"]["tied"] == tied
    gm = gw.model(max_seq_len=0, max_sequences=2)          # 0: the file's context_length
    assert gm.max_seq_len == 32 and gm.cfg["qkv_bias"] == bias
    om = _oracle_model(orc, cfg, W, 32, 2)
    ids = [3, 17, 42, 8, 8, 29, 499]
    for pos, t in enumerate(ids):
        hid, log = gm.forward_token(1, pos, t)
        want_h = om.token_forward(1, pos, t)
        close(hid, want_h, 5e-3, 5e-3 * max(1.0, np.abs(want_h).max()))     # whole-layer tolerance, tests/forward_parity_toy.rs:389
        assert int(np.argmax(log)) == int(np.argmax(om.logits(want_h)))
    got, gap = gm.decode_greedy(0, ids, 12)
    om.alloc_kv(32, 2)
    want, _ = om.decode_greedy(0, ids, 12)
    print(f"[{arch}/{naming}] min top-2 logit gap {gap.min():.3e}")
    assert np.array_equal(got, want)
    # the same weights uploaded array by array: identical ids (same kernels, different addresses)
    dm = syn.DeviceModel(ctx, cfg, W, max_seq_len=32, max_sequences=2)
    assert np.array_equal(dm.decode_greedy(0, ids, 12)[0], got)
    dm.close()
    gm.close()
    gw.close()


def test_layer_without_norm_tensors_runs_the_unweighted_norm(ctx, orc, tmpfile):
    # forward.rs:317-325: no norm tensor -> plain RMS norm; the loader substitutes a weight of ones
    cfg = dict(n_layers=2, d_model=64, q_heads=4, kv_heads=4, head_dim=16, ffn=128, vocab=200, rms_eps=1e-5, rope_base=10000.0,
               rope_scale=1.0, rope_layout=0, qkv_bias=False, context_length=16)
    W = syn.make_weights(cfg, seed=9, std=0.1, emb_std=1.0)
    W["ffn_norm"][0] = (1 + 0.2 * np.random.default_rng(1).standard_normal(64)).astype(np.float32)
    data = model_file(cfg, W, drop=("blk.1.attn_norm.weight", "blk.1.ffn_norm.weight"))
    gw = gg.GgufWeights(ctx, tmpfile(data))
    assert gw.info["layers"][1]["attn_norm"] is None and gw.info["layers"][0]["attn_norm"] is not None
    gm = gw.model(16, 1)
    om = _oracle_model(orc, cfg, W, 16, 1)                  # W holds ones for the dropped tensors
    got, _ = gm.decode_greedy(0, [5, 6, 7], 8)
    want, _ = om.decode_greedy(0, [5, 6, 7], 8)
    assert np.array_equal(got, want)
    gm.close()
    gw.close()


def test_hot_path_shapes_from_a_file(ctx, orc, tmpfile):
    # d_model 2048 (the shape the fused kernels are tuned for), two layers, ~200 MB file
    cfg = dict(n_layers=2, d_model=2048, q_heads=32, kv_heads=4, head_dim=64, ffn=5632, vocab=1000, rms_eps=1e-5,
               rope_base=10000.0, rope_scale=1.0, rope_layout=0, qkv_bias=False, context_length=64)
    W = syn.make_weights(cfg, seed=2, std=0.03, emb_std=1.0)
    gw = gg.GgufWeights(ctx, tmpfile(model_file(cfg, W)))
    gm = gw.model(64, 4)
    om = _oracle_model(orc, cfg, W, 64, 4)
    prompt = [1, 22, 333, 4]
    for mode in (0, 2):                                      # the reference's call sequence, then fused + graph replay
        gm.set_mode(mode)
        got, gap = gm.decode_greedy(0, prompt, 6)
        om.alloc_kv(64, 4)
        want, _ = om.decode_greedy(0, prompt, 6)
        assert np.array_equal(got, want), f"mode {mode}, min gap {gap.min():.3e}"
    # batched step over the same file-resident weights
    seqs, first, second = [1, 2, 3], [7, 8, 9], [70, 80, 90]
    for s, t in zip(seqs, first):
        gm.forward_token(s, 0, t, want_hidden=False, want_logits=False)
    ids, _ = gm.decode_batch_greedy(seqs, [1, 1, 1], second, 4)
    for r, s in enumerate(seqs):
        om.alloc_kv(64, 4)
        want, _ = om.decode_greedy(s, [first[r], second[r]], 4)
        assert np.array_equal(ids[r], want[2:]), f"row {r}"
    gm.close()
    gw.close()


def test_files_this_build_does_not_run_are_refused_with_a_reason(ctx, tmpfile):
    cfg = dict(n_layers=1, d_model=64, q_heads=4, kv_heads=4, head_dim=16, ffn=128, vocab=64, rms_eps=1e-5, rope_base=10000.0,
               rope_scale=1.0, rope_layout=0, qkv_bias=False, context_length=16)
    W = syn.make_weights(cfg, seed=1)
    gw = gg.GgufWeights(ctx, tmpfile(model_file(cfg, W, drop=("output_norm.weight",))))
    with pytest.raises(gg.GgufError, match="output norm tensor not found"):
        gw.model(16, 1)
    gw.close()
    gw = gg.GgufWeights(ctx, tmpfile(model_file(cfg, W, drop=("blk.0.ffn_down.weight",))))
    with pytest.raises(gg.GgufError, match="mapping standard layer 0: missing required tensor"):
        gw.model(16, 1)
    gw.close()
    # a descriptor that points outside the data section: rejected before anything is allocated or copied
    bad = llama_metadata(GgufWriter()).tensor("W", [4, 8], F16_T, offset=0).build_raw(b"\0" * 63)
    with pytest.raises(gg.GgufError, match="overflows weights blob"):
        gg.GgufWeights(ctx, tmpfile(bad))
    with pytest.raises(gg.GgufError, match="Not a GGUF file"):
        gg.GgufWeights(ctx, tmpfile(b"not a gguf file at all"))
    lib = ctx.lib
    import ctypes as C
    p = C.c_void_p()
    assert lib.m40llm_ext_upload_file_range(ctx.h, b"/nonexistent", 0, 16, C.byref(p)) == -6
    path = tmpfile(b"0123456789abcdef")
    assert lib.m40llm_ext_upload_file_range(ctx.h, path.encode(), 8, 9, C.byref(p)) == -6     # range ends outside the file
    assert lib.m40llm_ext_upload_file_range(None, path.encode(), 0, 8, C.byref(p)) == -1
    assert lib.m40llm_ext_upload_file_range(ctx.h, path.encode(), 4, 8, C.byref(p)) == 0
    out = np.empty(8, dtype=np.uint8)
    assert lib.m40llm_memcpy_d2h(ctx.h, out.ctypes.data_as(C.c_void_p), p, 8) == 0 and out.tobytes() == b"456789ab"
    assert lib.m40llm_device_free(ctx.h, p) == 0
