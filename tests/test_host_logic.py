"""Host layer (C++ mirror of the reference's decode / batch / sampling / KV-config / telemetry modules),
checked against the literals in the reference's own unit tests.  No GPU needed: nothing here computes on the device."""
import ctypes as C
import importlib
import os
import subprocess

import numpy as np
import pytest

m40 = importlib.import_module("m40-llm_amd")


@pytest.fixture(scope="module")
def H():
    return m40.host()


def fptr(a):
    return np.ascontiguousarray(a, dtype=np.float32).ctypes.data_as(C.c_void_p)


def u32(a):
    return np.ascontiguousarray(a, dtype=np.uint32)


# ---------------------------------------------------------------- C ABI surface
def test_native_library_exports_every_declared_symbol():
    lib = m40.native()      # loads without a GPU
    protos = m40.parse_header(m40.HEADER)
    out = subprocess.check_output(["nm", "-D", "--defined-only", m40.NATIVE_LIB], text=True)
    exported = {l.split()[-1] for l in out.splitlines() if " T " in l}
    assert len(protos) >= 91
    missing = sorted(set(protos) - exported)
    assert not missing, missing
    for name in protos:
        assert getattr(lib, name) is not None
    assert b"gfx950" in lib.m40llm_ext_build_info()


def test_surface_covers_the_reference_stub_symbols():
    """The reference's non-CUDA stub (cuda/stub.c), compiled as-is, lists the names its FFI binds."""
    ref = os.path.join(m40.ROOT, "oracle", "_ref", "libm40llm_refstub.so")
    if not os.path.exists(ref):
        pytest.skip("reference stub witness not built (reference checkout absent)")
    names = lambda p: {l.split()[-1] for l in subprocess.check_output(["nm", "-D", "--defined-only", p], text=True).splitlines()
                       if " T m40llm_" in l}
    assert len(names(ref)) == 80
    assert names(ref) <= names(m40.NATIVE_LIB)


def test_unavailable_symbols_report_minus_one_without_a_device():
    lib = m40.native()
    assert lib.m40llm_start_persistent_decode(None) == -1
    assert lib.m40llm_gemm_f32xf32_f32_async(None, None, None, None, 1, 1, 1) == -1
    assert lib.m40llm_attention_prefill_f32_gqa_varlen(None, None, None, None, None, None, None, None, 1, 1, 1, 64, None) == -1   # null arguments
    # argument checks that run before any device work
    assert lib.m40llm_device_malloc(None, 16, None) == -1
    assert lib.m40llm_gemm_f32xf16_gguf_f32(None, None, None, None, 1, 1, 1) == -1
    assert lib.m40llm_rms_norm_f32_async(None, None, None, 1, 8, 1e-5) == -1
    assert lib.m40llm_validate_device_ptr(None) == -1
    assert lib.m40llm_stream_synchronize(None, 1) == -1


# ---------------------------------------------------------------- sampling (src/sampling.rs tests)
def test_sampler_reference_cases(H):
    s = H.m40host_sampler_create(1.0, -1, 0.0, 42)
    assert H.m40host_sampler_sample_greedy(s, fptr([0.1, -0.2, 5.0, 1.0]), 4) == 2
    for _ in range(10):   # NaN entry zeroed, the rest sampled; the reference asserts index 2 ten times with seed 42
        assert H.m40host_sampler_sample(s, fptr([np.nan, -1.0, 3.0]), 3) == 2
    H.m40host_sampler_destroy(s)
    s = H.m40host_sampler_create(1.0, 1, 0.0, 42)
    for _ in range(100):
        assert H.m40host_sampler_sample(s, fptr([0.0, 5.0, 1.0]), 3) == 1
    assert H.m40host_sampler_sample(s, fptr([2.0, 2.0, 1.0]), 3) == 0          # stable order: lowest index wins ties
    assert H.m40host_sampler_sample(s, fptr([-np.inf, -np.inf]), 2) == 0
    H.m40host_sampler_destroy(s)
    s = H.m40host_sampler_create(0.5, -1, 0.0, 42)
    c1 = sum(H.m40host_sampler_sample(s, fptr([0.0, 1.0]), 2) == 1 for _ in range(1000))
    assert c1 > 600
    H.m40host_sampler_destroy(s)
    s = H.m40host_sampler_create(1.0, -1, 0.60, 123)
    for _ in range(100):
        assert H.m40host_sampler_sample(s, fptr([0.0, 1.0, 2.0]), 3) in (1, 2)
    H.m40host_sampler_destroy(s)
    a = H.m40host_sampler_create(0.9, -1, 0.0, 7); b = H.m40host_sampler_create(0.9, -1, 0.0, 7)
    la = [H.m40host_sampler_sample(a, fptr([0.5, 0.25, 0.25]), 3) for _ in range(10)]
    lb = [H.m40host_sampler_sample(b, fptr([0.5, 0.25, 0.25]), 3) for _ in range(10)]
    assert la == lb
    assert H.m40host_sampler_sample(a, fptr([]), 0) == -1 and b"empty logits" in H.m40host_last_error()
    H.m40host_sampler_destroy(a); H.m40host_sampler_destroy(b)


def test_sampler_xorshift_stream_and_topk1_matches_oracle(H, orc):
    # xorshift64* with seed 42: first outputs computed independently in Python integers
    state = 42
    def nxt():
        nonlocal state
        x = state
        x ^= x >> 12; x ^= (x << 25) & 0xFFFFFFFFFFFFFFFF; x ^= x >> 27
        state = x
        return (x * 0x2545F4914F6CDD1D) & 0xFFFFFFFFFFFFFFFF
    # a uniform two-way choice consumes one draw per call: index = 0 iff r <= 0.5
    s = H.m40host_sampler_create(1.0, -1, 0.0, 42)
    for _ in range(50):
        r = np.float32(nxt() >> 41) / np.float32(1 << 23)
        r = np.float32(r * np.float32(1.0))
        want = 0 if r <= np.float32(0.5) else 1
        assert H.m40host_sampler_sample(s, fptr([1.0, 1.0]), 2) == want
    H.m40host_sampler_destroy(s)
    rng = np.random.default_rng(0)
    g = H.m40host_greedy_sampler(123)
    for _ in range(50):
        logits = rng.standard_normal(997).astype(np.float32)
        assert H.m40host_sampler_sample(g, fptr(logits), 997) == orc.greedy_topk1(logits) == int(np.argmax(logits))
    H.m40host_sampler_destroy(g)


# ---------------------------------------------------------------- stopping / decode loop
def test_stopping_criteria_reference_cases(H):
    z = u32([])
    stop = lambda mt, eos, gen: H.m40host_should_stop(mt, eos, z.ctypes.data_as(C.c_void_p), 0, 0, u32(gen).ctypes.data_as(C.c_void_p), len(gen))
    assert [stop(3, -1, g) for g in ([], [1], [1, 2], [1, 2, 3])] == [0, 0, 0, 1]      # tests/decode_stopping.rs
    assert [stop(-1, 42, g) for g in ([], [1, 2], [1, 2, 42])] == [0, 0, 1]
    assert [stop(5, 9, g) for g in ([1, 2, 3], [1, 2, 3, 4, 5], [1, 9])] == [0, 1, 1]
    ids = u32([7, 3, 7])
    assert H.m40host_should_stop(-1, -1, ids.ctypes.data_as(C.c_void_p), 3, 1, u32([5, 3]).ctypes.data_as(C.c_void_p), 2) == 1
    assert H.m40host_should_stop(-1, -1, ids.ctypes.data_as(C.c_void_p), 3, 1, u32([5, 4]).ctypes.data_as(C.c_void_p), 2) == 0


def test_decode_loop_respects_eos_and_max_tokens(H):
    # tests/decode_loop.rs: logits spike cycles 'H','i','!' with eos '!' and max 5 -> ids end with H, i, !
    seq = [ord("H"), ord("i"), ord("!")]
    calls = {"n": 0}
    CB = C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(C.c_uint32), C.c_size_t, C.POINTER(C.c_float), C.c_size_t)

    def cb(user, ids, n_ids, out, vocab):
        for i in range(vocab):
            out[i] = 0.0
        out[seq[calls["n"] % 3]] = 100.0
        calls["n"] += 1
        return 0
    cbp = CB(cb)
    s = H.m40host_greedy_sampler(123)
    out = np.zeros(64, dtype=np.uint32)
    z = u32([])
    n = H.m40host_decode_loop(z.ctypes.data_as(C.c_void_p), 0, s, 5, ord("!"), z.ctypes.data_as(C.c_void_p), 0, 0, 256, C.cast(cbp, C.c_void_p), None,
                              out.ctypes.data_as(C.c_void_p), 64)
    assert n == 3 and list(out[:3]) == seq
    # max_tokens wins when no eos is hit; prompt ids are kept in front
    calls["n"] = 0
    s2 = H.m40host_greedy_sampler(123)
    n = H.m40host_decode_loop(u32([9, 8]).ctypes.data_as(C.c_void_p), 2, s2, 2, -1, z.ctypes.data_as(C.c_void_p), 0, 0, 256, C.cast(cbp, C.c_void_p), None,
                              out.ctypes.data_as(C.c_void_p), 64)
    assert n == 4 and list(out[:4]) == [9, 8, ord("H"), ord("i")]
    H.m40host_sampler_destroy(s); H.m40host_sampler_destroy(s2)


# ---------------------------------------------------------------- pool / batch plan
def test_sequence_pool_leases_and_returns_slots(H):
    pool = H.m40host_pool_create(2)          # src/decode_batch.rs:362-378
    assert H.m40host_pool_capacity(pool) == 2 and H.m40host_pool_available(pool) == 2
    first = H.m40host_pool_try_lease(pool); second = H.m40host_pool_try_lease(pool)
    assert H.m40host_lease_sequence_id(first) == 0 and H.m40host_lease_sequence_id(second) == 1
    assert H.m40host_pool_available(pool) == 0 and H.m40host_pool_try_lease(pool) is None
    H.m40host_lease_release(first)
    assert H.m40host_pool_available(pool) == 1
    third = H.m40host_pool_try_lease(pool)
    assert H.m40host_lease_sequence_id(third) == 0
    H.m40host_lease_release(second); H.m40host_lease_release(third)
    # FIFO free list: slots come back in release order
    a = H.m40host_pool_try_lease(pool)
    assert H.m40host_lease_sequence_id(a) == 1
    H.m40host_lease_release(a)
    H.m40host_pool_destroy(pool)


def _plan(H, reqs):
    rid = np.array([r[0] for r in reqs], dtype=np.uint64); sid = u32([r[1] for r in reqs])
    kvl = u32([r[2] for r in reqs]); st = u32([r[3] for r in reqs])
    return H.m40host_batch_plan_from_requests(rid.ctypes.data_as(C.c_void_p), sid.ctypes.data_as(C.c_void_p), kvl.ctypes.data_as(C.c_void_p), st.ctypes.data_as(C.c_void_p), len(reqs))


def test_decode_batch_keeps_active_mixed_lengths(H):
    # src/decode_batch.rs:381-397
    p = _plan(H, [(10, 2, 5, 0), (11, 3, 7, 1), (12, 4, 1, 0), (13, 5, 9, 2), (14, 6, 3, 0)])
    assert p and H.m40host_batch_plan_size(p) == 3
    ids = np.zeros(3, dtype=np.uint32); lens = np.zeros(3, dtype=np.uint32)
    H.m40host_batch_plan_sequence_ids(p, ids.ctypes.data_as(C.c_void_p)); H.m40host_batch_plan_sequence_lens(p, lens.ctypes.data_as(C.c_void_p))
    assert list(ids) == [2, 4, 6] and list(lens) == [5, 1, 3]
    assert H.m40host_batch_plan_total_q_tokens(p) == 3 and H.m40host_batch_plan_total_kv_tokens(p) == 9
    assert H.m40host_batch_plan_total_attention_cells(p) == 9
    assert H.m40host_batch_plan_query_len(p, 0) == 1
    assert H.m40host_batch_plan_index_for_request(p, 12) == 1 and H.m40host_batch_plan_index_for_request(p, 11) == -1
    assert H.m40host_batch_plan_output_offset_f32(p, 14, 4, 64) == 2 * 4 * 64 == 512
    H.m40host_batch_plan_destroy(p)
    assert _plan(H, [(1, 0, 1, 1)]) is None and b"at least one active request" in H.m40host_last_error()
    assert _plan(H, [(1, 0, 0, 0)]) is None and b"zero kv_len" in H.m40host_last_error()


def test_batch_metadata_prefix_offsets_and_validation(H):
    tq, tkv, cells = C.c_uint32(), C.c_uint32(), C.c_uint64()
    chk = lambda s, k, q: H.m40host_batch_metadata_check(u32(s).ctypes.data_as(C.c_void_p), u32(k).ctypes.data_as(C.c_void_p), u32(q).ctypes.data_as(C.c_void_p), len(s),
                                                         C.byref(tq), C.byref(tkv), C.byref(cells))
    assert chk([7, 3, 128], [7, 9, 128], [7, 1, 16]) == 0      # tests/batch_metadata.rs
    assert (tq.value, tkv.value, cells.value) == (24, 144, 2106)
    assert chk([], [], []) == -1 and b"at least one sequence" in H.m40host_last_error()
    assert chk([0], [1], [1]) == -1 and b"zero seq_len" in H.m40host_last_error()
    assert chk([4], [4], [0]) == -1 and b"zero query_len" in H.m40host_last_error()
    assert chk([4], [0], [1]) == -1 and b"zero kv_len" in H.m40host_last_error()
    assert chk([2], [4], [3]) == -1 and b"exceeds seq_len" in H.m40host_last_error()
    assert chk([4], [1], [2]) == -1 and b"smaller than query_len" in H.m40host_last_error()
    assert chk([0xFFFFFFFF, 1], [1, 1], [1, 1]) == -1 and b"overflow" in H.m40host_last_error()


# ---------------------------------------------------------------- KV compression config (src/kv_compression.rs:326-427)
class KvCfg(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("mode", "recent_window", "block_size", "top_blocks", "representatives",
                                           "representative_policy", "exact_old_backing", "exact_old_attention")]

    def as_tuple(self):
        return tuple(getattr(self, f[0]) for f in self._fields_)


OFF, BSE = 0, 2
DENSE, Q8, FP16KQ4V = 0, 1, 2
STAGED, Q8DIRECT, Q4DIRECT = 0, 1, 2


def _val(H, c, rt=None):
    err = C.create_string_buffer(512)
    rc = (H.m40host_kvcfg_validate(C.byref(c), err, 512) if rt is None
          else H.m40host_kvcfg_validate_runtime_support(C.byref(c), rt[0], rt[1], err, 512))
    return rc, err.value.decode()


def test_kv_compression_config_reference_cases(H, monkeypatch):
    monkeypatch.delenv("M40LLM_KV_EXACT_OLD_BACKING", raising=False)
    monkeypatch.delenv("M40LLM_KV_EXACT_OLD_ATTENTION", raising=False)
    d = KvCfg(); H.m40host_kvcfg_default(C.byref(d))
    assert d.as_tuple() == (BSE, 1024, 32, 8, 0, 0, FP16KQ4V, Q4DIRECT)
    assert _val(H, d)[0] == 0 and _val(H, d, (2048, 64))[0] == 0 and _val(H, d, (2048, 128))[0] == 0
    r = KvCfg(); H.m40host_kvcfg_dense_reference(C.byref(r))
    assert r.as_tuple() == (OFF, 1024, 32, 8, 0, 0, DENSE, STAGED)
    assert _val(H, r)[0] == 0 and _val(H, r, (16, 128))[0] == 0
    rc, msg = _val(H, d, (512, 64)); assert rc == -1 and "kv_recent_window" in msg
    q8 = KvCfg(); H.m40host_kvcfg_default(C.byref(q8)); q8.exact_old_backing = Q8; q8.exact_old_attention = Q8DIRECT
    rc, msg = _val(H, q8, (2048, 128)); assert rc == -1 and "head_dim=128" in msg
    t = KvCfg(); H.m40host_kvcfg_default(C.byref(t)); t.top_blocks = 65
    rc, msg = _val(H, t, (2048, 64)); assert rc == -1 and "limit of 64" in msg
    mm = KvCfg(); H.m40host_kvcfg_dense_reference(C.byref(mm)); mm.mode = BSE; mm.exact_old_attention = Q4DIRECT
    rc, msg = _val(H, mm); assert rc == -1 and "requires kv_exact_old_backing" in msg
    mo = KvCfg(); H.m40host_kvcfg_dense_reference(C.byref(mo)); mo.exact_old_backing = FP16KQ4V
    rc, msg = _val(H, mo); assert rc == -1 and "requires kv_compress_mode" in msg
    z = KvCfg(); H.m40host_kvcfg_default(C.byref(z)); z.recent_window = 0
    assert "kv_recent_window must be > 0" in _val(H, z)[1]
    z.recent_window = 4; z.block_size = 0
    assert "kv_compress_block must be > 0" in _val(H, z)[1]
    z.block_size = 4; z.top_blocks = 0
    assert "top_blocks must be > 0" in _val(H, z)[1]
    fm = KvCfg(); H.m40host_kvcfg_for_mode(BSE, C.byref(fm)); assert fm.as_tuple() == d.as_tuple()
    H.m40host_kvcfg_for_mode(3, C.byref(fm)); assert fm.as_tuple() == (3, 1024, 32, 8, 0, 0, DENSE, STAGED)
    # environment override only applies while the field is at its Dense / Staged default
    monkeypatch.setenv("M40LLM_KV_EXACT_OLD_BACKING", "fp16-k-q4-v")
    monkeypatch.setenv("M40LLM_KV_EXACT_OLD_ATTENTION", "direct-fp16-k-q4-v")
    e = KvCfg(); H.m40host_kvcfg_dense_reference(C.byref(e)); e.mode = BSE
    assert H.m40host_kvcfg_effective_backing(C.byref(e)) == FP16KQ4V and H.m40host_kvcfg_effective_attention(C.byref(e)) == Q4DIRECT
    assert H.m40host_kvcfg_effective_backing(C.byref(q8)) == Q8


def test_scoped_runtime_config_shadows_global_config(H):
    r = KvCfg(); H.m40host_kvcfg_dense_reference(C.byref(r))
    H.m40host_kvcfg_set_runtime(C.byref(r))
    s = KvCfg(); H.m40host_kvcfg_default(C.byref(s)); s.top_blocks = 4
    g = H.m40host_kvcfg_scoped_push(C.byref(s))
    cur = KvCfg(); H.m40host_kvcfg_get_runtime(C.byref(cur)); assert cur.as_tuple() == s.as_tuple()
    H.m40host_kvcfg_scoped_pop(g)
    H.m40host_kvcfg_get_runtime(C.byref(cur)); assert cur.as_tuple() == r.as_tuple()


# ---------------------------------------------------------------- selection telemetry
def test_kv_selection_recorder(H, monkeypatch):
    monkeypatch.delenv("M40LLM_KV_SELECTION_TELEMETRY", raising=False)
    monkeypatch.delenv("M40LLM_KV_ATTENTION_CAPTURE", raising=False)
    H.m40host_kvsel_reset()
    assert H.m40host_kvsel_enabled() == 0
    n_sel, total, top, n_rec = C.c_size_t(), C.c_uint32(), C.c_uint32(), C.c_size_t()
    sel = np.zeros(16, dtype=np.uint32)
    assert H.m40host_kvsel_snapshot(sel.ctypes.data_as(C.c_void_p), 16, C.byref(n_sel), C.byref(total), C.byref(top), C.byref(n_rec)) == 0
    H.m40host_kvsel_set_attention_context(3, 17)
    H.m40host_kvsel_record_scored_timed(u32([5, 2]).ctypes.data_as(C.c_void_p), fptr([0.9, 0.5]), u32([160, 64]).ctypes.data_as(C.c_void_p),
                                        u32([192, 96]).ctypes.data_as(C.c_void_p), 2, 10, 8, 1.5)
    H.m40host_kvsel_set_attention_context(-1, -1)
    H.m40host_kvsel_record(u32([2, 7]).ctypes.data_as(C.c_void_p), 2, 12, 4)
    assert H.m40host_kvsel_snapshot(sel.ctypes.data_as(C.c_void_p), 16, C.byref(n_sel), C.byref(total), C.byref(top), C.byref(n_rec)) == 1
    assert list(sel[: n_sel.value]) == [2, 5, 7] and (total.value, top.value, n_rec.value) == (12, 8, 2)   # maxima, sorted set
    layer, token, n, rt, rtop, el = C.c_int64(), C.c_int64(), C.c_size_t(), C.c_uint32(), C.c_uint32(), C.c_float()
    ranks = np.zeros(8, dtype=np.uint32); blocks = np.zeros(8, dtype=np.uint32); scores = np.zeros(8, dtype=np.float32)
    st = np.zeros(8, dtype=np.uint32); en = np.zeros(8, dtype=np.uint32)
    assert H.m40host_kvsel_snapshot_record(0, C.byref(layer), C.byref(token), ranks.ctypes.data_as(C.c_void_p), blocks.ctypes.data_as(C.c_void_p),
                                           scores.ctypes.data_as(C.c_void_p), st.ctypes.data_as(C.c_void_p), en.ctypes.data_as(C.c_void_p), 8, C.byref(n), C.byref(rt),
                                           C.byref(rtop), C.byref(el)) == 0
    assert (layer.value, token.value, n.value, rt.value, rtop.value, el.value) == (3, 17, 2, 10, 8, 1.5)
    assert list(ranks[:2]) == [0, 1] and list(blocks[:2]) == [5, 2] and list(st[:2]) == [160, 64] and list(en[:2]) == [192, 96]
    assert H.m40host_kvsel_snapshot_record(1, C.byref(layer), C.byref(token), None, blocks.ctypes.data_as(C.c_void_p), scores.ctypes.data_as(C.c_void_p),
                                           None, None, 8, C.byref(n), None, None, C.byref(el)) == 0
    assert (layer.value, token.value, el.value) == (-1, -1, -1.0) and list(scores[:2]) == [0.0, 0.0]
    # capture policy
    monkeypatch.setenv("M40LLM_KV_SELECTION_TELEMETRY", "yes")
    assert H.m40host_kvsel_enabled() == 1
    assert H.m40host_kvsel_should_capture_attention() == 1           # default policy "first", nothing captured yet
    H.m40host_kvsel_record_attention(0.7, 0.3)
    assert H.m40host_kvsel_should_capture_attention() == 0
    H.m40host_kvsel_record_attention(0.6, 0.4)
    assert H.m40host_kvsel_attention_count() == 1
    monkeypatch.setenv("M40LLM_KV_ATTENTION_CAPTURE", "layer:2, token:9")
    H.m40host_kvsel_set_attention_context(2, 8); assert H.m40host_kvsel_should_capture_attention() == 0
    H.m40host_kvsel_set_attention_context(2, 9); assert H.m40host_kvsel_should_capture_attention() == 1
    monkeypatch.setenv("M40LLM_KV_ATTENTION_CAPTURE", "ALL")
    H.m40host_kvsel_record_attention(0.5, 0.5)
    assert H.m40host_kvsel_attention_count() == 2
    H.m40host_kvsel_reset()
    assert H.m40host_kvsel_snapshot(sel.ctypes.data_as(C.c_void_p), 16, C.byref(n_sel), C.byref(total), C.byref(top), C.byref(n_rec)) == 0
