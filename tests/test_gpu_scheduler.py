"""Continuous batching on the GPU: requests that arrive at different ticks, share batched prefill and decode steps and
reuse sequence slots generate exactly the tokens the CPU oracle generates for each of them alone."""
import importlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from gpu_common import m40  # noqa: E402
from test_gpu_model import _assert_ids_equal_up_to_legitimate_tie, _oracle_greedy_with_logits  # noqa: E402

syn = importlib.import_module("m40-llm_amd.synthetic")
sch = importlib.import_module("m40-llm_amd.scheduler")


@pytest.fixture(scope="module")
def ctx():
    yield m40.Context(0)


@pytest.mark.parametrize("mode,hd", [(2, 64), (0, 64), (2, 16)])      # head_dim 16: no packed prefill, prompts go token by token
def test_scheduler_outputs_equal_oracle_greedy_per_request(ctx, orc, mode, hd):
    cfg = dict(n_layers=2, d_model=4 * hd if hd >= 64 else 256, q_heads=4 if hd >= 64 else 16, kv_heads=2, head_dim=hd, ffn=512,
               vocab=300, rms_eps=1e-5, rope_base=10000.0, rope_scale=1.0, rope_layout=0, qkv_bias=False)
    W = syn.make_weights(cfg, seed=12, std=0.08, emb_std=1.0)
    dm = syn.DeviceModel(ctx, cfg, W, max_seq_len=64, max_sequences=3)
    dm.set_mode(mode)
    om = orc.Model(dict(cfg, qkv_bias=False), W)
    rng = np.random.default_rng(4)
    specs = [(rng.integers(0, 300, size=n).tolist(), g) for n, g in ((9, 7), (1, 12), (20, 3), (5, 6), (2, 9))]
    s = sch.Scheduler.for_model(dm)
    rids = {}
    pending = list(enumerate(specs))
    ticks = 0
    while pending or s.active():
        # two arrivals at the start, then one more whenever a slot is free
        while pending and s.available_slots() and (ticks > 0 or len(rids) < 2):
            i, (prompt, gen) = pending.pop(0)
            rids[i] = s.submit(prompt, max_tokens=gen)
            if ticks > 0:
                break
        s.tick()
        ticks += 1
        assert ticks < 200
    for i, (prompt, gen) in enumerate(specs):
        om.alloc_kv(64, 1)
        want, gaps = om.decode_greedy(0, prompt, gen)
        assert s.state(rids[i]) == "complete", s.error(rids[i])
        assert s.generated(rids[i]) == want[len(prompt):].tolist(), (i, float(gaps.min()))
    assert s.available_slots() == 3
    s.close()
    dm.close()


def test_scheduler_full_depth_tinyllama_requests_equal_oracle(ctx, orc, heartbeat):
    """The scheduler at the full BASELINE config-2 shape (22 layers): six requests with prompts of 40-150 tokens on four
    slots, arrivals spread over the ticks, so that packed prefills of one to three prompts, batched decode steps of one to
    four rows with device-side picks, and reused slots all occur.  Each request's tokens equal what the oracle generates
    for it alone -- its prompt through the oracle's packed prefill, as the scheduler runs prompts
    (src/server.rs:420-560 -> forward.rs:2153-2600), then token by token -- up to a listed tie."""
    cfg = dict(syn.TINYLLAMA_1B)
    W = syn.make_weights(cfg, seed=0)
    S, n_new = 192, 12
    dm = syn.DeviceModel(ctx, cfg, W, max_seq_len=S, max_sequences=4)
    dm.set_mode(2)
    om = orc.Model(dict(cfg, qkv_bias=False), W)
    orc.set_threads(16)
    rng = np.random.default_rng(11)
    specs = [rng.integers(0, cfg["vocab"], size=n).tolist() for n in (150, 40, 97, 64, 120, 41)]
    s = sch.Scheduler.for_model(dm)
    rids, pending, ticks = {}, list(enumerate(specs)), 0
    while pending or s.active():
        # three arrivals at the start (one packed prefill of three prompts), later ones as slots free up, two at a time
        burst = 3 if ticks == 0 else 2
        while pending and s.available_slots() and burst and (ticks == 0 or ticks % 5 == 0):
            i, prompt = pending.pop(0)
            rids[i] = s.submit(prompt, max_tokens=n_new)
            burst -= 1
        s.tick()
        ticks += 1
        assert ticks < 400
    for i, prompt in enumerate(specs):
        assert s.state(rids[i]) == "complete", s.error(rids[i])
        om.alloc_kv(S, 1)
        hidden = om.prefill_forward([0], [prompt])[-1]
        want, wgap, wscale = _oracle_greedy_with_logits(orc, om, 0, [], n_new, start_pos=len(prompt), hidden=hidden)
        heartbeat()
        _assert_ids_equal_up_to_legitimate_tie(s.generated(rids[i]), want, wgap, wscale, f"scheduler, 22 layers, request {i} (prompt of {len(prompt)})")
    assert s.available_slots() == 4
    s.close()
    dm.close()
