"""Continuous batching on the GPU: requests that arrive at different ticks, share batched prefill and decode steps and
reuse sequence slots generate exactly the tokens the CPU oracle generates for each of them alone."""
import importlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from gpu_common import m40  # noqa: E402

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
