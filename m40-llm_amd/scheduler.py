"""ctypes view of the host layer's continuous-batching decode scheduler (m40host_scheduler_* in
include/m40llm_host.h; the reference's server scheduler, src/server.rs:203-770, without HTTP and tokenizer)."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import host

STATES = {0: "unknown", 1: "pending_prefill", 2: "decoding", 3: "complete", 4: "cancelled", 5: "failed"}

PREFILL_FN = C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.c_uint32,
                         C.POINTER(C.c_float))
DECODE_FN = C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.c_uint32,
                        C.POINTER(C.c_float))


class TickReport(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("prefill_rows", "prefill_tokens", "decode_rows", "completed", "cancelled", "failed")]


class SchedulerError(RuntimeError):
    pass


class Scheduler:
    """for_model(device_model) drives a model; with_engine(...) takes Python callbacks
    prefill(seq_ids, prompts) -> logits [batch][vocab] and decode(seq_ids, kv_lens, tokens) -> logits [rows][vocab]."""

    def __init__(self, handle, keep=()):
        self.H = host()
        self.h = handle
        self._keep = keep
        if not self.h:
            raise SchedulerError(self.H.m40host_last_error().decode())

    @classmethod
    def for_model(cls, model, sequence_slots: int = 0):
        H = host()
        return cls(H.m40host_scheduler_create_for_model(model.h, sequence_slots), keep=(model,))

    @classmethod
    def with_engine(cls, vocab: int, max_seq_len: int, sequence_slots: int, prefill, decode):
        H = host()

        def _prefill(_user, seqs, lens, toks, batch, out):
            try:
                seq_ids = [seqs[i] for i in range(batch)]
                prompts, at = [], 0
                for i in range(batch):
                    prompts.append([toks[at + j] for j in range(lens[i])])
                    at += lens[i]
                logits = np.ascontiguousarray(prefill(seq_ids, prompts), dtype=np.float32).reshape(batch, vocab)
                C.memmove(out, logits.ctypes.data, logits.nbytes)
                return 0
            except Exception:
                return 1

        def _decode(_user, seqs, lens, toks, rows, out):
            try:
                logits = np.ascontiguousarray(decode([seqs[i] for i in range(rows)], [lens[i] for i in range(rows)],
                                                     [toks[i] for i in range(rows)]), dtype=np.float32).reshape(rows, vocab)
                C.memmove(out, logits.ctypes.data, logits.nbytes)
                return 0
            except Exception:
                return 1

        pf, df = PREFILL_FN(_prefill), DECODE_FN(_decode)
        h = H.m40host_scheduler_create_with_engine(vocab, max_seq_len, sequence_slots, C.cast(pf, C.c_void_p), C.cast(df, C.c_void_p), None)
        return cls(h, keep=(pf, df))

    def close(self):
        if getattr(self, "h", None):
            self.H.m40host_scheduler_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def submit(self, prompt, max_tokens: int = -1, stop_ids=(), temperature: float = 1.0, top_k: int = 1, top_p: float = 0.0,
               seed: int = 42) -> int:
        p = np.ascontiguousarray(prompt, dtype=np.uint32)
        s = np.ascontiguousarray(list(stop_ids), dtype=np.uint32)
        rid = self.H.m40host_scheduler_submit(self.h, p.ctypes.data_as(C.c_void_p), len(p), max_tokens,
                                              s.ctypes.data_as(C.c_void_p) if len(s) else None, len(s), temperature, top_k, top_p, seed)
        if rid < 0:
            raise SchedulerError(self.H.m40host_last_error().decode())
        return rid

    def cancel(self, rid: int) -> bool:
        return bool(self.H.m40host_scheduler_cancel(self.h, rid))

    def tick(self) -> TickReport:
        rep = TickReport()
        if self.H.m40host_scheduler_tick(self.h, C.byref(rep)) != 0:
            raise SchedulerError(self.H.m40host_last_error().decode())
        return rep

    def state(self, rid: int) -> str:
        return STATES[self.H.m40host_scheduler_state(self.h, rid)]

    def sequence_of(self, rid: int) -> int:
        return self.H.m40host_scheduler_sequence_of(self.h, rid)

    def active(self) -> int:
        return self.H.m40host_scheduler_active(self.h)

    def available_slots(self) -> int:
        return self.H.m40host_scheduler_available_slots(self.h)

    def generated(self, rid: int) -> list:
        n = self.H.m40host_scheduler_generated(self.h, rid, None, 0)
        out = np.zeros(max(n, 1), dtype=np.uint32)
        self.H.m40host_scheduler_generated(self.h, rid, out.ctypes.data_as(C.c_void_p), n)
        return out[:n].tolist()

    def error(self, rid: int) -> str:
        buf = C.create_string_buffer(512)
        self.H.m40host_scheduler_error(self.h, rid, buf, 512)
        return buf.value.decode()

    def run_until_idle(self, max_ticks: int = 100000) -> int:
        ticks = 0
        while self.active() and ticks < max_ticks:
            self.tick()
            ticks += 1
        return ticks
