"""The step function: one batch of (request, its next tokens) through the model.

A step runs only the tokens it is given, from the cache that earlier steps
left: portions of prompts beside single decoded tokens, cut anywhere.  It
returns the logits at the places that are asked for.  The reference's
counterpart is ``model_forward`` with the six step tensors
(src/exec/model.rs:62-85, src/exec/cache_scheduler/mod.rs:824-930); here the
wanted rows are arbitrary, not only each sequence's last.

Steps that hold nothing but single decoded tokens, each wanting its logits, can
be replayed from a captured HIP graph: the same forward pass, recorded once per
(number of rows, block-table width) and fed through fixed device buffers.  The
reference does the same around its forward (python/vosti_kernels/graph_overlay.py:177-389):
a signature runs eagerly when first seen, is captured when seen again, and is
replayed from then on.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from ..cache import CachePool
from ..kernels.ops import ATTN_ITEM_ROWS, SEGMENT_KEYS
from ..parts.base import GroupTables, StepContext

WIDTH_BUCKET = 8       # captured block tables grow in steps of this many pages
# Captured decode steps have one of these numbers of rows; a step with fewer is filled up with rows that
# read one key of page 0 and write nothing (the reference pads its graphs likewise,
# python/vosti_kernels/graph_overlay.py:177-389).
ROW_BUCKETS = (1, 2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64, 96, 128, 192, 256, 384, 512)


@dataclass
class StepEntry:
    request_id: int
    tokens: list[int]
    want: list[int] = field(default_factory=list)   # places among ``tokens`` whose logits are wanted


@dataclass
class _Layout:
    """Host arrays of one step and where each lies in the one buffer that is uploaded."""
    parts: list[np.ndarray]
    offsets: list[int]
    total: int
    q_lens: list[int]
    starts: list[int]
    max_k_len: int
    max_decode_k_len: int

    def pack(self, out: np.ndarray) -> None:
        for p, o in zip(self.parts, self.offsets):
            out[o:o + p.size] = p.reshape(-1)


@dataclass
class _Captured:
    graph: torch.cuda.CUDAGraph
    meta: torch.Tensor        # the device buffer the graph reads
    staging: torch.Tensor     # pinned host twin
    logits: torch.Tensor      # the graph's output
    copied: torch.cuda.Event  # the last upload from ``staging``


class ModelRunner:
    """Binds a model to a cache pool and runs steps."""

    def __init__(self, model, pool: CachePool, graphs: bool = False):
        self.model, self.pool, self.cache = model, pool, pool.manager
        self.kernels = model.kernels
        self.graphs = graphs
        self._scratch: torch.Tensor | None = None
        self._seen: set[tuple] = set()
        self._captured: dict[tuple, _Captured] = {}
        self._keepalive: list[torch.Tensor] = []
        self.graph_stats = {"eager": 0, "captured": 0, "replayed": 0}

    # ---------------------------------------------------------------- pieces
    def _attn_scratch(self, n_floats: int) -> torch.Tensor:
        if self._scratch is None or self._scratch.numel() < n_floats:
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError("the attention scratch buffer must be sized before a graph is captured")
            if self._scratch is not None and self._captured:
                self._keepalive.append(self._scratch)      # captured graphs still point at it
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

    def _layout(self, entries: list[StepEntry], widths: list[int] | None = None, rows: int | None = None) -> _Layout:
        """The step's host arrays.  ``widths``: block-table width per group (default: what the step needs).
        ``rows``: fill up to this many sequences with padding rows of one token: token 0 at position 0,
        one key (whatever page 0 holds), slot -1 (nothing is stored), logits wanted like the others."""
        cache, spec = self.cache, self.model.spec
        real = len(entries)
        S = max(real, rows or 0)
        q_lens = [len(e.tokens) for e in entries] + [1] * (S - real)
        T = sum(q_lens)
        starts = []
        for e, n in zip(entries, q_lens):
            if cache.pending(e.request_id) != n:
                raise RuntimeError(f"request {e.request_id}: the cache holds pages for {cache.pending(e.request_id)} "
                                   f"pending tokens, the step brings {n}")
            starts.append(cache.length(e.request_id))
        starts += [0] * (S - real)
        ids = np.concatenate([np.asarray(e.tokens, dtype=np.int64) for e in entries] + [np.zeros(S - real, dtype=np.int64)])
        if ids.min() < 0 or ids.max() >= spec.vocab_size:
            raise ValueError(f"token id out of range [0, {spec.vocab_size})")
        k_len = np.asarray([s + n for s, n in zip(starts, q_lens)], dtype=np.int32)
        if int(k_len.max()) > spec.max_positions:
            raise ValueError(f"a request would reach {int(k_len.max())} tokens; the model's positions end at {spec.max_positions}")
        positions = np.concatenate([np.arange(s, s + n, dtype=np.int32) for s, n in zip(starts, q_lens)])
        cu_q = np.zeros(S + 1, dtype=np.int32)
        np.cumsum(q_lens, out=cu_q[1:])
        state_slots = np.asarray([cache.state_slot(e.request_id) for e in entries] + [0] * (S - real), dtype=np.int32)
        want = []
        for e, base, n in zip(entries, cu_q[:-1], q_lens):
            for w in e.want:
                if not 0 <= w < n:
                    raise ValueError(f"request {e.request_id}: wanted place {w} is outside its {n} tokens")
                want.append(int(base) + w)
        want += [int(cu_q[s]) for s in range(real, S)]
        prefill_items, decode_items = [], []
        for s, n in enumerate(q_lens):
            if n == 1:
                decode_items.append((s, 0))
            else:
                prefill_items.extend((s, off) for off in range(0, n, ATTN_ITEM_ROWS))
        parts: list[np.ndarray] = [ids.astype(np.int32), positions, cu_q, k_len, state_slots,
                                   np.asarray(want, dtype=np.int32),
                                   np.asarray(prefill_items, dtype=np.int32).reshape(-1, 2),
                                   np.asarray(decode_items, dtype=np.int32).reshape(-1, 2)]
        for g in range(len(self.pool.group_windows)):
            width = widths[g] if widths else self.needed_width(entries, g)
            table = np.zeros((S, width), dtype=np.int32)
            slots = np.full(T, -1, dtype=np.int32)
            for s, e in enumerate(entries):
                cache.block_table_row(e.request_id, g, width, table[s])
                cache.slots(e.request_id, g, starts[s], q_lens[s], slots[cu_q[s]:cu_q[s + 1]])
            parts += [slots, table]
        # One buffer, one copy; every piece starts on a 16-byte boundary.
        offsets, total = [], 0
        for p in parts:
            offsets.append(total)
            total += (p.size + 3) & ~3
        dec_k = [int(k_len[s]) for s, n in enumerate(q_lens) if n == 1]
        return _Layout(parts, offsets, max(total, 4), q_lens, starts, int(k_len.max()), max(dec_k) if dec_k else 0)

    def needed_width(self, entries: list[StepEntry], group: int) -> int:
        return max(1, max(self.cache.num_logical_pages(e.request_id, group) for e in entries))

    def _context(self, lay: _Layout, dev: torch.Tensor, max_k_len: int, max_decode_k_len: int):
        views = [dev[o:o + p.size].view(p.shape) for p, o in zip(lay.parts, lay.offsets)]
        ids_d, pos_d, cu_d, klen_d, slots_d, want_d, pre_d, dec_d = views[:8]
        groups = [GroupTables(slots=views[8 + 2 * g], block_table=views[9 + 2 * g], window=w)
                  for g, w in enumerate(self.pool.group_windows)]
        ctx = StepContext(kernels=self.kernels, num_tokens=sum(lay.q_lens), num_seqs=len(lay.q_lens), positions=pos_d,
                          cu_q=cu_d, k_len=klen_d, state_slots=slots_d, groups=groups, prefill_items=pre_d,
                          decode_items=dec_d, max_k_len=max_k_len, max_decode_k_len=max_decode_k_len,
                          host_q_lens=lay.q_lens, host_starts=lay.starts, host_state_slots=lay.parts[4].tolist(),
                          attn_scratch=self._attn_scratch)
        return ids_d, ctx, want_d

    def build_context(self, entries: list[StepEntry]):
        """Host arrays of the step -> one upload -> (ids, context, wanted rows)."""
        lay = self._layout(entries)
        host = np.zeros(lay.total, dtype=np.int32)
        lay.pack(host)
        return self._context(lay, torch.from_numpy(host).to("cuda"), lay.max_k_len, lay.max_decode_k_len)

    # ---------------------------------------------------------------- running
    def run(self, entries: list[StepEntry]) -> torch.Tensor:
        """The forward pass of a step whose pages are taken; logits [wanted, vocab] in the element type."""
        if self.graphs and all(len(e.tokens) == 1 and e.want == [0] for e in entries):
            return self._run_decode_graph(entries)
        self.graph_stats["eager"] += 1
        ids, ctx, want = self.build_context(entries)
        return self.model.forward(ids, ctx, self.pool.entries, want)

    def _run_decode_graph(self, entries: list[StepEntry]) -> torch.Tensor:
        P = self.pool.page_size
        widths = [-(-self.needed_width(entries, g) // WIDTH_BUCKET) * WIDTH_BUCKET
                  for g in range(len(self.pool.group_windows))]
        # A mixer with state of its own would have to be told which rows are padding: no padding then.
        rows = len(entries) if self.pool.has_state else next((b for b in ROW_BUCKETS if b >= len(entries)), len(entries))
        key = (rows, tuple(widths))
        cap = self._captured.get(key)
        if cap is None and key not in self._seen:
            # First sight of a signature: eagerly, which also warms up every kernel it uses.
            self._seen.add(key)
            self.graph_stats["eager"] += 1
            ids, ctx, want = self.build_context(entries)
            return self.model.forward(ids, ctx, self.pool.entries, want)
        lay = self._layout(entries, widths, rows)
        # Launch geometry is frozen in the graph: it must cover every length the tables can hold.
        cover = min(max(widths) * P, self.model.spec.max_positions)
        if cap is None:
            self._attn_scratch(self._max_scratch(rows, cover))
            staging = torch.empty(lay.total, dtype=torch.int32, pin_memory=True)
            meta = torch.zeros(lay.total, dtype=torch.int32, device="cuda")
            lay.pack(staging.numpy())
            meta.copy_(staging, non_blocking=True)
            ids, ctx, want = self._context(lay, meta, cover, cover)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                logits = self.model.forward(ids, ctx, self.pool.entries, want)
            cap = _Captured(graph, meta, staging, logits, torch.cuda.Event())
            self._captured[key] = cap
            self.graph_stats["captured"] += 1
        else:
            cap.copied.synchronize()                       # the staging buffer is free again
            lay.pack(cap.staging.numpy())
            cap.meta.copy_(cap.staging, non_blocking=True)
        cap.copied.record()
        cap.graph.replay()
        self.graph_stats["replayed"] += 1
        return cap.logits[:len(entries)]

    def _max_scratch(self, tokens: int, cover: int) -> int:
        """Floats of attention scratch that any mixer of the model needs for ``tokens`` decode rows over ``cover`` keys."""
        nseg = -(-cover // SEGMENT_KEYS)
        need = 1
        for block in self.model.layers:
            m = block.mixer
            if hasattr(m, "nq") and hasattr(m, "d"):
                need = max(need, self.kernels.attn_scratch_floats(tokens, m.nq, m.d, nseg))
        return need

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
