"""The step function: one batch of (request, its next tokens) through the model.

A step runs only the tokens it is given, from the cache that earlier steps
left: portions of prompts beside single decoded tokens, cut anywhere.  It
returns the logits at the places that are asked for.  The reference's
counterpart is ``model_forward`` with the six step tensors
(src/exec/model.rs:62-85, src/exec/cache_scheduler/mod.rs:824-930); here the
wanted rows are arbitrary, not only each sequence's last.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from ..cache import CachePool
from ..parts.base import GroupTables, StepContext

ROW_TILE = 16   # rows of one attention work item


@dataclass
class StepEntry:
    request_id: int
    tokens: list[int]
    want: list[int] = field(default_factory=list)   # places among ``tokens`` whose logits are wanted


class ModelRunner:
    """Binds a model to a cache pool and runs steps."""

    def __init__(self, model, pool: CachePool):
        self.model, self.pool, self.cache = model, pool, pool.manager
        self.kernels = model.kernels
        self._scratch: torch.Tensor | None = None

    # ---------------------------------------------------------------- pieces
    def _attn_scratch(self, n_floats: int) -> torch.Tensor:
        if self._scratch is None or self._scratch.numel() < n_floats:
            self._scratch = torch.empty(max(n_floats, 1 << 16), dtype=torch.float32, device="cuda")
        return self._scratch

    def begin(self, entries: list[StepEntry]) -> None:
        """Takes the pages of the step's tokens (and a state slot for new requests)."""
        done = []
        try:
            for e in entries:
                if not e.tokens:
                    raise ValueError(f"request {e.request_id}: a step entry needs at least one token")
                if not self.cache.has_request(e.request_id):
                    self.cache.add_request(e.request_id)
                self.cache.extend(e.request_id, e.tokens)
                done.append(e.request_id)
        except Exception:
            for rid in done:
                self.cache.abort_step(rid)
            raise

    def end(self, entries: list[StepEntry]) -> None:
        for e in entries:
            self.cache.commit(e.request_id)

    def build_context(self, entries: list[StepEntry]) -> tuple[torch.Tensor, StepContext, torch.Tensor]:
        """Host arrays of the step -> one upload -> (ids, context, wanted rows)."""
        cache, spec = self.cache, self.model.spec
        S = len(entries)
        q_lens = [len(e.tokens) for e in entries]
        T = sum(q_lens)
        starts = []
        for e, n in zip(entries, q_lens):
            if cache.pending(e.request_id) != n:
                raise RuntimeError(f"request {e.request_id}: the cache holds pages for {cache.pending(e.request_id)} "
                                   f"pending tokens, the step brings {n}")
            starts.append(cache.length(e.request_id))
        ids = np.concatenate([np.asarray(e.tokens, dtype=np.int64) for e in entries])
        if ids.min() < 0 or ids.max() >= spec.vocab_size:
            raise ValueError(f"token id out of range [0, {spec.vocab_size})")
        k_len = np.asarray([s + n for s, n in zip(starts, q_lens)], dtype=np.int32)
        if int(k_len.max()) > spec.max_positions:
            raise ValueError(f"a request would reach {int(k_len.max())} tokens; the model's positions end at {spec.max_positions}")
        positions = np.concatenate([np.arange(s, s + n, dtype=np.int32) for s, n in zip(starts, q_lens)])
        cu_q = np.zeros(S + 1, dtype=np.int32)
        np.cumsum(q_lens, out=cu_q[1:])
        state_slots = np.asarray([cache.state_slot(e.request_id) for e in entries], dtype=np.int32)
        want = []
        for e, base, n in zip(entries, cu_q[:-1], q_lens):
            for w in e.want:
                if not 0 <= w < n:
                    raise ValueError(f"request {e.request_id}: wanted place {w} is outside its {n} tokens")
                want.append(int(base) + w)
        prefill_items, decode_items = [], []
        for s, n in enumerate(q_lens):
            if n == 1:
                decode_items.append((s, 0))
            else:
                prefill_items.extend((s, off) for off in range(0, n, ROW_TILE))
        parts: list[np.ndarray] = [ids.astype(np.int32), positions, cu_q, k_len, state_slots,
                                   np.asarray(want, dtype=np.int32),
                                   np.asarray(prefill_items, dtype=np.int32).reshape(-1, 2),
                                   np.asarray(decode_items, dtype=np.int32).reshape(-1, 2)]
        n_groups = len(self.pool.group_windows)
        for g in range(n_groups):
            width = max(1, max(cache.num_logical_pages(e.request_id, g) for e in entries))
            table = np.zeros((S, width), dtype=np.int32)
            slots = np.empty(T, dtype=np.int32)
            for s, e in enumerate(entries):
                cache.block_table_row(e.request_id, g, width, table[s])
                cache.slots(e.request_id, g, starts[s], q_lens[s], slots[cu_q[s]:cu_q[s + 1]])
            parts += [slots, table]
        # One buffer, one copy; every piece starts on a 16-byte boundary.
        offsets, total = [], 0
        for p in parts:
            offsets.append(total)
            total += (p.size + 3) & ~3
        host = np.zeros(max(total, 4), dtype=np.int32)
        for p, o in zip(parts, offsets):
            host[o:o + p.size] = p.reshape(-1)
        dev = torch.from_numpy(host).to("cuda")
        views = [dev[o:o + p.size].view(p.shape) for p, o in zip(parts, offsets)]
        ids_d, pos_d, cu_d, klen_d, slots_d, want_d, pre_d, dec_d = views[:8]
        groups = [GroupTables(slots=views[8 + 2 * g], block_table=views[9 + 2 * g], window=self.pool.group_windows[g])
                  for g in range(n_groups)]
        dec_k = [int(k_len[s]) for s, n in enumerate(q_lens) if n == 1]
        ctx = StepContext(kernels=self.kernels, num_tokens=T, num_seqs=S, positions=pos_d, cu_q=cu_d, k_len=klen_d,
                          state_slots=slots_d, groups=groups, prefill_items=pre_d, decode_items=dec_d,
                          max_k_len=int(k_len.max()), max_decode_k_len=max(dec_k) if dec_k else 0,
                          host_q_lens=q_lens, host_starts=starts, attn_scratch=self._attn_scratch)
        return ids_d, ctx, want_d

    def run(self, entries: list[StepEntry]) -> torch.Tensor:
        """The forward pass of a step whose pages are taken; logits [wanted, vocab] in the element type."""
        ids, ctx, want = self.build_context(entries)
        return self.model.forward(ids, ctx, self.pool.entries, want)

    # ------------------------------------------------------------------ whole
    def step(self, entries: list[StepEntry]) -> torch.Tensor:
        """Pages, forward, commit.  Logits of the wanted places, in the order of the entries and of ``want``."""
        if not entries:
            return self.kernels.empty(0, self.model.spec.vocab_size)
        if len({e.request_id for e in entries}) != len(entries):
            raise ValueError("a request appears twice in one step")
        self.begin(entries)
        try:
            logits = self.run(entries)
        except Exception:
            for e in entries:
                self.cache.abort_step(e.request_id)
            raise
        self.end(entries)
        return logits

    def finish(self, request_id: int) -> None:
        """The request is over: its pages and its slot go back."""
        self.cache.finish(request_id)
