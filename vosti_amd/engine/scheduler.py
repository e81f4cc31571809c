"""Python face of the native scheduler (csrc/host/scheduler.h)."""
from __future__ import annotations

import ctypes
from ctypes import c_int
from dataclasses import dataclass

import numpy as np

from ..cache.host import host_lib, i32_array
from ..cache.manager import CacheManager, OutOfPages

ADMISSION = ["Accepted", "DuplicateRequestId", "EmptyPrompt", "TooManyEosTokenIds", "ZeroMaxTokens",
             "HistoryCapacityOverflow", "EmptyEosTokenIds"]
PLAN_OK, PLAN_IDLE, PLAN_OUT_OF_PAGES, PLAN_STEP_PENDING, PLAN_INTERNAL = 0, 1, 2, 3, 4


class SchedulerError(RuntimeError):
    """The scheduler was driven out of order, or found the cache manager in a state it cannot plan from."""


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

    def add_request(self, request_id: int, prompt: list[int], max_tokens: int, eos_token_ids=(),
                    ignore_eos: bool | None = None) -> str:
        """Returns the admission status by name ('Accepted', 'EmptyPrompt', ...); only appends to the waiting queue.

        ``ignore_eos`` None: end tokens count if there are any.  False with no end token is refused as
        'EmptyEosTokenIds', as the reference refuses it (src/exec/engine.rs:2718-2720)."""
        if ignore_eos is None:
            ignore_eos = not eos_token_ids
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
        if st == PLAN_STEP_PENDING:
            raise SchedulerError("plan() before the step planned last was committed or given up (abort_step)")
        if st == PLAN_INTERNAL:
            raise SchedulerError("the cache manager refused a planned row for a reason other than pages")
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
        """The planned step ran: one sampled token per sampled row, in row order."""
        n = self._lib.vh_sched_commit(self._h, i32_array(sampled) if sampled else None, len(sampled))
        if n < 0:
            raise SchedulerError(f"commit() got {len(sampled)} sampled tokens for a plan with "
                                 f"{self._lib.vh_sched_num_planned_samples(self._h)} sampled rows; nothing was committed")
        out = np.empty((n, 3), dtype=np.int64)
        if n:
            self._lib.vh_sched_get_emitted(self._h, out.ctypes.data)
        return [Emitted(r, t, bool(f)) for r, t, f in out.tolist()]

    def abort_step(self) -> None:
        """The planned step did not run: its rows' tokens stay uncomputed and the next plan() decides again."""
        self._lib.vh_sched_abort_step(self._h)

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
