"""The tensors behind the cache manager's numbers.

From the model's cache needs (one per schedule entry) the pool forms the groups
of the cache manager (one per distinct window; every all-keys layer shares group
0's page indices, as in the reference where one block id indexes the same page
in every layer: python/vosti_kernels/physical.py:139-147), allocates K and V
pages per entry and a row of state per slot for mixers with state, and hands each
schedule entry the object its mixer expects.
"""
from __future__ import annotations

import torch

from ..parts.base import KVPagesSpec, PagedKV, StateSlotSpec, StateSlots
from .manager import CacheManager, GroupSpec


class CachePool:
    def __init__(self, model, *, page_size: int, num_pages: int, num_slots: int, prefix_cache: bool = False,
                 window_pages: int | None = None):
        """``num_pages``: pages of every all-keys group.  ``window_pages``: pages of every
        windowed group (default: the same number)."""
        if page_size < 8 or page_size & (page_size - 1):
            raise ValueError(f"page size {page_size} must be a power of two, at least 8")
        specs = model.cache_specs()
        self.page_size = page_size
        windows: list[int] = []
        for s in specs:
            if isinstance(s, KVPagesSpec) and s.window not in windows:
                windows.append(s.window)
        windows.sort()          # 0 (all keys) first
        if not windows:
            windows = [0]
        has_state = any(isinstance(s, StateSlotSpec) for s in specs)
        self.has_state = has_state
        groups = [GroupSpec(w, num_pages if w == 0 else (window_pages or num_pages)) for w in windows]
        # A prefix page holds keys only; a mixer with state of its own could not resume from it.
        self.manager = CacheManager(page_size, groups, num_slots, prefix_cache and not has_state)
        self.group_windows = windows
        dtype = model.kernels.dtype
        self.entries: list = []
        for i, (entry, s) in enumerate(zip(model.schedule, specs)):
            if entry.cache_from is not None:
                src = self.entries[entry.cache_from]
                if not isinstance(src, PagedKV):
                    raise ValueError(f"schedule entry {i} reads the cache of entry {entry.cache_from}, which keeps no pages")
                self.entries.append(PagedKV(src.k, src.v, src.group, page_size, writable=False))
            elif isinstance(s, KVPagesSpec):
                g = windows.index(s.window)
                n = groups[g].num_pages
                k = torch.zeros(n, s.num_kv_heads, page_size, s.head_dim, dtype=dtype, device="cuda")
                v = torch.zeros(n, s.num_kv_heads, s.head_dim, page_size, dtype=dtype, device="cuda")
                self.entries.append(PagedKV(k, v, g, page_size))
            elif isinstance(s, StateSlotSpec):
                self.entries.append(StateSlots(torch.zeros(num_slots, *s.shape, dtype=s.dtype, device="cuda")))
            elif s is None:
                self.entries.append(None)
            else:
                raise ValueError(f"schedule entry {i}: unknown cache need {s!r}")

    def bytes(self) -> int:
        seen, total = set(), 0
        for e in self.entries:
            for t in ((e.k, e.v) if isinstance(e, PagedKV) else (e.state,) if isinstance(e, StateSlots) else ()):
                if t.data_ptr() not in seen:
                    seen.add(t.data_ptr())
                    total += t.numel() * t.element_size()
        return total
