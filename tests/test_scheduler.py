"""Continuous-batching decode scheduler (host logic, no GPU): a deterministic fake engine behind the callback
interface checks that every request receives exactly the tokens it would get decoding alone, that each engine call
carries the right cache lengths and tokens for its slot, and the slot-pool, cancellation, stopping and failure rules of
the reference's server scheduler (src/server.rs:203-770, src/decode_batch.rs:14-85)."""
import importlib

import numpy as np
import pytest

sch = importlib.import_module("m40-llm_amd.scheduler")

VOCAB = 97


def next_token(history):
    return (sum(history) * 31 + len(history) * 7 + 3) % VOCAB


def logits_for(history):
    rng = np.random.default_rng(len(history) * 1000003 + sum(history))
    out = rng.standard_normal(VOCAB).astype(np.float32)
    out[next_token(history)] = 9.0
    return out


class FakeEngine:
    """Keeps the token history of every sequence slot, as a KV cache would, and checks what the scheduler sends."""

    def __init__(self):
        self.hist = {}
        self.calls = []
        self.fail_next = False

    def prefill(self, seq_ids, prompts):
        if self.fail_next:
            self.fail_next = False
            raise RuntimeError("injected")
        assert len(set(seq_ids)) == len(seq_ids)
        self.calls.append(("prefill", list(seq_ids), [len(p) for p in prompts]))
        for s, p in zip(seq_ids, prompts):
            self.hist[s] = list(p)                     # a prefill starts the slot over at position 0
        return np.stack([logits_for(self.hist[s]) for s in seq_ids])

    def decode(self, seq_ids, kv_lens, tokens):
        if self.fail_next:
            self.fail_next = False
            raise RuntimeError("injected")
        assert len(set(seq_ids)) == len(seq_ids)
        self.calls.append(("decode", list(seq_ids), list(kv_lens)))
        for s, n, t in zip(seq_ids, kv_lens, tokens):
            assert n == len(self.hist[s]), (s, n, len(self.hist[s]))     # the token's position = tokens already cached
            self.hist[s].append(t)
        return np.stack([logits_for(self.hist[s]) for s in seq_ids])


def alone(prompt, max_tokens, stop_ids=()):
    """What one request generates when it decodes by itself (src/decode.rs:60-100)."""
    ids, gen = list(prompt), []
    while len(gen) < max_tokens and not (gen and gen[-1] in stop_ids):
        t = next_token(ids)
        ids.append(t)
        gen.append(t)
    return gen


def make(slots=4, max_seq_len=64):
    eng = FakeEngine()
    return eng, sch.Scheduler.with_engine(VOCAB, max_seq_len, slots, eng.prefill, eng.decode)


def test_requests_batched_together_generate_what_they_would_alone():
    eng, s = make()
    prompts = [[1, 2, 3], [50], [9, 8, 7, 6, 5, 4], [11, 12]]
    budgets = [5, 1, 9, 3]
    rids = [s.submit(p, max_tokens=b) for p, b in zip(prompts, budgets)]
    assert rids == [1, 2, 3, 4] and [s.sequence_of(r) for r in rids] == [0, 1, 2, 3] and s.available_slots() == 0
    rep = s.tick()
    assert (rep.prefill_rows, rep.prefill_tokens, rep.decode_rows, rep.completed) == (4, 12, 0, 1)    # the 1-token budget is done
    assert s.state(2) == "complete" and s.state(1) == "decoding"
    rep = s.tick()
    assert (rep.prefill_rows, rep.decode_rows) == (0, 3)
    ticks = 2 + s.run_until_idle()
    assert ticks == max(budgets)                                  # the prefill tick samples token 1, each decode tick one more
    for r, p, b in zip(rids, prompts, budgets):
        assert s.state(r) == "complete" and s.generated(r) == alone(p, b)
    assert s.available_slots() == 4 and s.active() == 0
    assert eng.calls[0] == ("prefill", [0, 1, 2, 3], [3, 1, 6, 2])
    assert eng.calls[1] == ("decode", [0, 2, 3], [3, 6, 2])       # the finished request left the batch


def test_arrivals_join_running_batches_and_slots_are_reused_in_fifo_order():
    eng, s = make(slots=2)
    a = s.submit([1, 2, 3], max_tokens=6)
    b = s.submit([4], max_tokens=2)
    with pytest.raises(sch.SchedulerError, match="sequence lease"):
        s.submit([5], max_tokens=2)                                  # pool exhausted: refused, nothing queues
    s.tick()                                                         # prefill a, b
    s.tick()                                                         # decode a, b; b reaches its budget
    assert s.state(b) == "complete" and s.available_slots() == 1    # its lease went back with it
    c = s.submit([7, 7, 7, 7], max_tokens=4, stop_ids=[next_token([7, 7, 7, 7])])   # stops on its first token
    assert s.sequence_of(c) == 1                                     # the freed slot
    rep = s.tick()
    assert (rep.prefill_rows, rep.decode_rows, rep.completed) == (1, 1, 1) and s.state(c) == "complete"
    s.run_until_idle()
    assert s.generated(a) == alone([1, 2, 3], 6) and s.generated(b) == alone([4], 2)
    assert s.generated(c) == alone([7, 7, 7, 7], 4, stop_ids=[next_token([7, 7, 7, 7])]) and len(s.generated(c)) == 1
    # free list is FIFO (src/decode_batch.rs:75-85): slots came back in the order 1 (b), 1 (c), 0 (a) -> next leases 1 then 0
    d, e = s.submit([1]), s.submit([2])
    assert (s.sequence_of(d), s.sequence_of(e)) == (1, 0)


def test_cancellation_failure_and_context_window():
    eng, s = make(slots=3, max_seq_len=6)
    a = s.submit([1, 2], max_tokens=50)
    b = s.submit([3, 4], max_tokens=50)
    s.tick()
    assert s.cancel(b) and not s.cancel(999)
    rep = s.tick()
    assert rep.cancelled == 1 and rep.decode_rows == 1 and s.state(b) == "cancelled" and len(s.generated(b)) == 1
    s.run_until_idle()
    # a holds 2 prompt + 4 generated tokens in a 6-token window when the next step would not fit
    assert s.state(a) == "failed" and "context window" in s.error(a) and s.generated(a) == alone([1, 2], 5)
    assert s.available_slots() == 3
    c = s.submit([5], max_tokens=3)
    eng.fail_next = True
    rep = s.tick()
    assert rep.failed == 1 and s.state(c) == "failed" and "batched prefill forward failed" in s.error(c)
    d = s.submit([5], max_tokens=3)
    s.tick()
    eng.fail_next = True
    s.tick()
    assert s.state(d) == "failed" and "batched decode forward failed" in s.error(d) and s.available_slots() == 3
    with pytest.raises(sch.SchedulerError, match="empty prompt"):
        s.submit([])
    with pytest.raises(sch.SchedulerError, match="context window"):
        s.submit([1] * 7)
    with pytest.raises(sch.SchedulerError, match="out of range"):
        s.submit([VOCAB])
    assert s.state(12345) == "unknown"


def test_sampling_requests_are_reproducible_per_seed():
    outs = []
    for _ in range(2):
        eng, s = make()
        r1 = s.submit([1, 2, 3], max_tokens=8, temperature=1.3, top_k=-1, top_p=0.9, seed=7)
        r2 = s.submit([1, 2, 3], max_tokens=8, temperature=1.3, top_k=-1, top_p=0.9, seed=8)
        s.run_until_idle()
        outs.append((s.generated(r1), s.generated(r2)))
    assert outs[0] == outs[1] and len(outs[0][0]) == 8
