"""Python face of the native cache manager (csrc/host/cache_manager.h).

It deals in integers only: which pages a request holds in each group of layers,
which state slot, how many tokens.  The tensors live in ``CachePool``.
"""
from __future__ import annotations

import ctypes
from ctypes import c_int
from dataclasses import dataclass

import numpy as np

from .host import host_lib, i32_array

OK, NO_PAGES, NO_SLOT, UNKNOWN_REQUEST, DUPLICATE_REQUEST, BAD_ARGUMENT, STEP_PENDING = range(7)
_STATUS = ["ok", "out of pages", "out of state slots", "unknown request", "duplicate request", "bad argument",
           "a step of this request is still pending"]


class CacheError(RuntimeError):
    pass


class OutOfPages(CacheError):
    pass


@dataclass(frozen=True)
class GroupSpec:
    window: int      # 0: all keys
    num_pages: int


class CacheManager:
    def __init__(self, page_size: int, groups: list[GroupSpec], num_slots: int, prefix_cache: bool = False):
        if page_size <= 0 or not groups:
            raise CacheError("the cache needs a positive page size and at least one group")
        self._lib = host_lib()
        self.page_size, self.groups, self.num_slots = page_size, list(groups), num_slots
        windows = (c_int * len(groups))(*[g.window for g in groups])
        pages = (c_int * len(groups))(*[g.num_pages for g in groups])
        self._h = self._lib.vh_cache_create(page_size, len(groups), windows, pages, num_slots, 1 if prefix_cache else 0)
        if not self._h:
            raise CacheError("bad cache geometry")
        self.prefix_cache = prefix_cache and all(g.window == 0 for g in groups)

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.vh_cache_destroy(h)

    @property
    def handle(self):
        return self._h

    def _raise(self, st: int, what: str):
        if st == NO_PAGES:
            raise OutOfPages(f"{what}: out of pages")
        raise CacheError(f"{what}: {_STATUS[st] if 0 <= st < len(_STATUS) else st}")

    # ------------------------------------------------------------ requests
    def add_request(self, rid: int, prompt: list[int] | None = None) -> int:
        """Takes a state slot; returns the number of prompt tokens found in the prefix cache."""
        cached = c_int(0)
        arr = i32_array(prompt) if prompt else None
        st = self._lib.vh_cache_add_request(self._h, rid, arr, len(prompt) if prompt else 0, ctypes.byref(cached))
        if st != OK:
            self._raise(st, f"add_request({rid})")
        return cached.value

    def reserve(self, rid: int, total_tokens: int) -> None:
        st = self._lib.vh_cache_reserve(self._h, rid, total_tokens)
        if st != OK:
            self._raise(st, f"reserve({rid}, {total_tokens})")

    def extend(self, rid: int, tokens: list[int]) -> None:
        st = self._lib.vh_cache_extend(self._h, rid, i32_array(tokens), len(tokens))
        if st != OK:
            self._raise(st, f"extend({rid}, {len(tokens)} tokens)")

    def try_extend(self, rid: int, tokens: list[int]) -> bool:
        st = self._lib.vh_cache_extend(self._h, rid, i32_array(tokens), len(tokens))
        if st == NO_PAGES:
            return False
        if st != OK:
            self._raise(st, f"extend({rid}, {len(tokens)} tokens)")
        return True

    def commit(self, rid: int) -> None:
        st = self._lib.vh_cache_commit(self._h, rid)
        if st != OK:
            self._raise(st, f"commit({rid})")

    def abort_step(self, rid: int) -> None:
        self._lib.vh_cache_abort_step(self._h, rid)

    def finish(self, rid: int) -> None:
        st = self._lib.vh_cache_finish(self._h, rid)
        if st != OK:
            self._raise(st, f"finish({rid})")

    # -------------------------------------------------------------- queries
    def has_request(self, rid: int) -> bool:
        return bool(self._lib.vh_cache_has_request(self._h, rid))

    def length(self, rid: int) -> int:
        return self._lib.vh_cache_length(self._h, rid)

    def pending(self, rid: int) -> int:
        return self._lib.vh_cache_pending(self._h, rid)

    def state_slot(self, rid: int) -> int:
        return self._lib.vh_cache_state_slot(self._h, rid)

    def num_logical_pages(self, rid: int, group: int) -> int:
        return self._lib.vh_cache_num_logical_pages(self._h, rid, group)

    def available_pages(self, group: int = 0) -> int:
        return self._lib.vh_cache_available_pages(self._h, group)

    def free_pages(self, group: int = 0) -> int:
        return self._lib.vh_cache_free_pages(self._h, group)

    def free_slots(self) -> int:
        return self._lib.vh_cache_free_slots(self._h)

    def num_requests(self) -> int:
        return self._lib.vh_cache_num_requests(self._h)

    def cached_blocks(self) -> int:
        return self._lib.vh_cache_cached_blocks(self._h)

    def drop_cached(self) -> int:
        """Gives every cached page that no request holds back to the free queue; returns how many."""
        return self._lib.vh_cache_drop_cached(self._h)

    def prefix_hits(self) -> int:
        return self._lib.vh_cache_prefix_hits(self._h)

    def prefix_hit_requests(self) -> int:
        """Admissions that found at least one cached page."""
        return self._lib.vh_cache_prefix_hit_requests(self._h)

    def evictions(self) -> int:
        return self._lib.vh_cache_evictions(self._h)

    def block_table_row(self, rid: int, group: int, width: int, out: np.ndarray | None = None) -> np.ndarray:
        out = np.empty(width, dtype=np.int32) if out is None else out
        st = self._lib.vh_cache_fill_block_table(self._h, rid, group, out.ctypes.data, width)
        if st != OK:
            self._raise(st, f"block_table_row({rid}, group {group}, width {width})")
        return out

    def slots(self, rid: int, group: int, start: int, n: int, out: np.ndarray | None = None) -> np.ndarray:
        out = np.empty(n, dtype=np.int32) if out is None else out
        st = self._lib.vh_cache_fill_slots(self._h, rid, group, start, n, out.ctypes.data)
        if st != OK:
            self._raise(st, f"slots({rid}, group {group}, {start}..{start + n})")
        return out

    def describe(self, rids: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
        """For the requests ``rids`` (uint64) in one call: [n, 3] = (committed length, pending tokens, state
        slot) and [n, groups] = the block-table width each needs."""
        n = rids.shape[0]
        out = np.empty((n, 3), dtype=np.int32)
        widths = np.empty((n, len(self.groups)), dtype=np.int32)
        st = self._lib.vh_cache_describe(self._h, n, rids.ctypes.data, out.ctypes.data, widths.ctypes.data)
        if st != OK:
            self._raise(st, "describe")
        return out, widths

    def fill_step(self, group: int, rids: np.ndarray, starts: np.ndarray, n_tokens: np.ndarray, table: np.ndarray,
                  slots: np.ndarray) -> None:
        """Block table rows (``table`` [rows >= n, width]; the rest reads page 0) and the slots of every token
        of the step (``slots`` [>= sum(n_tokens)]; the rest gets -1) of one group, in one call."""
        n = rids.shape[0]
        total = int(n_tokens.sum())
        st = self._lib.vh_cache_fill_step(self._h, group, n, rids.ctypes.data, starts.ctypes.data, n_tokens.ctypes.data,
                                          table.shape[0], table.shape[1], table.ctypes.data, slots.shape[0] - total,
                                          slots.ctypes.data)
        if st != OK:
            self._raise(st, f"fill_step(group {group})")

    def check(self) -> str:
        """'' if every page and slot is accounted for exactly once, else the first violation."""
        buf = ctypes.create_string_buffer(512)
        self._lib.vh_cache_check(self._h, buf, 512)
        return buf.value.decode()
