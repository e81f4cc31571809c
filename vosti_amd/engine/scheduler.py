"""Python face of the native scheduler (csrc/host/scheduler.h)."""
from __future__ import annotations

import ctypes
from ctypes import c_int
from dataclasses import dataclass

import numpy as np

from ..cache.host import host_lib, i32_array
from ..cache.manager import CacheManager, OutOfPages

ADMISSION = ["Accepted", "DuplicateRequestId", "EmptyPrompt", "TooManyEosTokenIds", "ZeroMaxTokens",
             "HistoryCapacityOverflow"]
PLAN_OK, PLAN_IDLE, PLAN_OUT_OF_PAGES = 0, 1, 2


@dataclass
class PlanRow:
    request_id: int
    start: int
    tokens: list[int]
    sample: bool
    state_slot: int
    output_index: int


@dataclass
class Emitted:
    request_id: int
    token: int
    finished: bool


class Scheduler:
    def __init__(self, cache: CacheManager, max_num_seqs: int, max_num_batched_tokens: int, max_model_len: int):
        self._lib = host_lib()
        self._cache = cache          # keeps the native manager alive
        self._h = self._lib.vh_sched_create(cache.handle, max_num_seqs, max_num_batched_tokens, max_model_len)
        if not self._h:
            raise ValueError("max_num_seqs, max_num_batched_tokens and max_model_len must be positive")
        self.max_num_seqs, self.max_num_batched_tokens = max_num_seqs, max_num_batched_tokens

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.vh_sched_destroy(h)

    def add_request(self, request_id: int, prompt: list[int], max_tokens: int, eos_token_ids=(), ignore_eos=False) -> str:
        """Returns the admission status by name ('Accepted', 'EmptyPrompt', ...); only appends to the waiting queue."""
        if len(eos_token_ids) > 3:
            return "TooManyEosTokenIds"
        st = self._lib.vh_sched_add_request(self._h, request_id, i32_array(prompt) if prompt else None, len(prompt),
                                            max_tokens, i32_array(list(eos_token_ids)) if eos_token_ids else None,
                                            len(eos_token_ids), 1 if ignore_eos else 0)
        return ADMISSION[st]

    def plan(self) -> list[PlanRow]:
        """Decides the next step and takes its pages.  [] when nothing is live."""
        n_rows, n_tokens = c_int(0), c_int(0)
        st = self._lib.vh_sched_plan(self._h, ctypes.byref(n_rows), ctypes.byref(n_tokens))
        if st == PLAN_OUT_OF_PAGES:
            raise OutOfPages("a request needs more cache pages than the pool has, even alone")
        if st == PLAN_IDLE or n_rows.value == 0:
            return []
        rows = np.empty((n_rows.value, 6), dtype=np.int64)
        toks = np.empty(n_tokens.value, dtype=np.int32)
        self._lib.vh_sched_get_plan(self._h, rows.ctypes.data, toks.ctypes.data)
        out, off = [], 0
        for rid, start, n, sample, slot, oi in rows.tolist():
            out.append(PlanRow(rid, start, toks[off:off + n].tolist(), bool(sample), slot, oi))
            off += n
        return out

    def commit(self, sampled: list[int]) -> list[Emitted]:
        n = self._lib.vh_sched_commit(self._h, i32_array(sampled) if sampled else None, len(sampled))
        out = np.empty((n, 3), dtype=np.int64)
        if n:
            self._lib.vh_sched_get_emitted(self._h, out.ctypes.data)
        return [Emitted(r, t, bool(f)) for r, t, f in out.tolist()]

    def abort(self, request_id: int) -> bool:
        return bool(self._lib.vh_sched_abort(self._h, request_id))

    def num_waiting(self) -> int:
        return self._lib.vh_sched_num_waiting(self._h)

    def num_running(self) -> int:
        return self._lib.vh_sched_num_running(self._h)

    def preemptions(self) -> int:
        return self._lib.vh_sched_preemptions(self._h)

    def is_live(self, request_id: int) -> bool:
        return bool(self._lib.vh_sched_is_live(self._h, request_id))
