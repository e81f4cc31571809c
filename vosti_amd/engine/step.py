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

from collections import OrderedDict
from dataclasses import dataclass, field

import numpy as np
import torch

from ..cache import CachePool
from ..cache.host import graph_row_bucket, graph_width_bucket, max_graphs as _max_graphs
from ..parts.base import GroupTables, HostStep, StepContext

# Captured decode steps have one of the numbers of rows 1, 2, 3, 4, 6, 8, 12, 16, ...; a step with fewer is filled
# up with rows that read one key of page 0 and write nothing (the reference pads its graphs likewise,
# python/vosti_kernels/graph_overlay.py:177-389).  Block tables are captured with one of these numbers times
# eight pages, so that a long generation walks through few captures.  The numbers, and how many graphs are
# kept, are the native library's (csrc/host/rules.h), which the native engine's step function uses too.
row_bucket = graph_row_bucket
width_bucket = graph_width_bucket


class GraphError(RuntimeError):
    """A capture or a replay failed: the runner replays nothing any more
    (python/vosti_kernels/graph_overlay.py:120-124, 173-175: no eager fallback after a failed replay)."""


@dataclass
class StepEntry:
    request_id: int
    tokens: list[int]
    want: list[int] = field(default_factory=list)   # places among ``tokens`` whose logits are wanted


@dataclass
class _Layout:
    """Host arrays of one step and where each lies in the one buffer that is uploaded."""
    parts: list[np.ndarray]
    names: list[str]            # names of the arrays that parts asked for (after the fixed ones)
    offsets: list[int]
    total: int
    host: HostStep

    def pack(self, out: np.ndarray) -> None:
        for p, o in zip(self.parts, self.offsets):
            out[o:o + p.size] = p.reshape(-1)


N_FIXED = 6      # ids, positions, cu_q, k_len, state slots, wanted rows


@dataclass
class _Captured:
    graph: torch.cuda.CUDAGraph
    meta: torch.Tensor        # the device buffer the graph reads
    staging: torch.Tensor     # pinned host twin
    logits: torch.Tensor      # the graph's output
    copied: torch.cuda.Event  # the last upload from ``staging``
    workspace: torch.Tensor   # the buffer its launches point into


class ModelRunner:
    """Binds a model to a cache pool and runs steps."""

    def __init__(self, model, pool: CachePool, graphs: bool = False, max_graphs: int | None = None):
        self.model, self.pool, self.cache = model, pool, pool.manager
        self.kernels = model.kernels
        self.max_graphs = max(1, int(_max_graphs() if max_graphs is None else max_graphs))   # the least recently replayed goes first
        self._workspace: torch.Tensor | None = None
        self._seen: set[tuple] = set()
        self._captured: "OrderedDict[tuple, _Captured]" = OrderedDict()
        self._graph_pool = None
        self._poisoned: str | None = None
        self.graph_stats = {"eager": 0, "captured": 0, "replayed": 0, "evicted": 0}
        # What the parts want of every step: one provider per distinct kind of per-step arrays.
        self._parts = list(model.parts())
        self.graphs = graphs and all(part.replayable for part in self._parts)
        self._providers = {}
        for part in self._parts:
            if part.step_inputs_key is not None:
                self._providers.setdefault(part.step_inputs_key, part)

    # ---------------------------------------------------------------- pieces
    def _get_workspace(self, n_floats: int) -> torch.Tensor:
        if self._workspace is None or self._workspace.numel() < n_floats:
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError("a part asks for more workspace inside a capture than it announced before it")
            # Captured graphs keep the buffer they were recorded with (``_Captured.workspace``).
            self._workspace = torch.empty(max(n_floats, 1 << 16), dtype=torch.float32, device="cuda")
        return self._workspace

    def workspace_needed(self, host: HostStep) -> int:
        return max((p.workspace_floats(host) for p in self._parts), default=0)

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

    def _layout(self, entries: list[StepEntry], widths: list[int] | None = None, rows: int | None = None,
                bound: int | None = None) -> _Layout:
        """The step's host arrays.  ``widths``: block-table width per group (default: what the step needs).
        ``rows``: fill up to this many sequences with padding rows of one token: token 0 at position 0,
        one key (whatever page 0 holds), slot -1 (nothing is stored), logits wanted like the others.
        ``bound``: the step is recorded for replay and its launches must cover this many keys."""
        cache, spec = self.cache, self.model.spec
        real = len(entries)
        S = max(real, rows or 0)
        pad = S - real
        rids = np.fromiter((e.request_id for e in entries), dtype=np.uint64, count=real)
        n_tok = np.fromiter((len(e.tokens) for e in entries), dtype=np.int32, count=real)
        info, needed = cache.describe(rids)              # one call for every request of the step
        if not np.array_equal(info[:, 1], n_tok):
            i = int(np.nonzero(info[:, 1] != n_tok)[0][0])
            raise RuntimeError(f"request {entries[i].request_id}: the cache holds pages for {int(info[i, 1])} "
                               f"pending tokens, the step brings {int(n_tok[i])}")
        starts_a = np.ascontiguousarray(info[:, 0])
        q_lens = n_tok.tolist() + [1] * pad
        starts = starts_a.tolist() + [0] * pad
        T = int(n_tok.sum()) + pad
        if T == S:                                       # one token each: no concatenation of lists
            ids = np.fromiter((e.tokens[0] for e in entries), dtype=np.int64, count=real)
            positions = starts_a.astype(np.int32)
        else:
            ids = np.concatenate([np.asarray(e.tokens, dtype=np.int64) for e in entries])
            positions = np.concatenate([np.arange(s, s + n, dtype=np.int32) for s, n in zip(starts, q_lens[:real])])
        if ids.min() < 0 or ids.max() >= spec.vocab_size:
            raise ValueError(f"token id out of range [0, {spec.vocab_size})")
        if pad:
            ids = np.concatenate([ids, np.zeros(pad, dtype=np.int64)])
            positions = np.concatenate([positions, np.zeros(pad, dtype=np.int32)])
        k_lens_a = np.concatenate([starts_a + n_tok, np.ones(pad, dtype=np.int32)]) if pad else starts_a + n_tok
        k_lens = k_lens_a.tolist()
        if int(k_lens_a.max()) > spec.max_positions:
            raise ValueError(f"a request would reach {int(k_lens_a.max())} tokens; the model's positions end at {spec.max_positions}")
        cu_q = np.zeros(S + 1, dtype=np.int32)
        np.cumsum(q_lens, out=cu_q[1:])
        state_slots = info[:, 2].tolist() + [0] * pad
        if all(e.want == [0] for e in entries) and T == S:
            want = cu_q[:-1].copy()
        else:
            want = []
            for e, base, n in zip(entries, cu_q[:-1], q_lens):
                for w in e.want:
                    if not 0 <= w < n:
                        raise ValueError(f"request {e.request_id}: wanted place {w} is outside its {n} tokens")
                    want.append(int(base) + w)
            want += [int(cu_q[s]) for s in range(real, S)]
            want = np.asarray(want, dtype=np.int32)
        host = HostStep(q_lens=q_lens, starts=starts, k_lens=k_lens, state_slots=state_slots,
                        k_len_bound=bound if bound is not None else max(k_lens), frozen=bound is not None)
        parts: list[np.ndarray] = [ids.astype(np.int32), positions, cu_q, k_lens_a.astype(np.int32, copy=False),
                                   np.asarray(state_slots, dtype=np.int32), want]
        for g in range(len(self.pool.group_windows)):
            width = widths[g] if widths else max(1, int(needed[:, g].max()))
            table = np.empty((S, width), dtype=np.int32)
            slots = np.empty(T, dtype=np.int32)
            cache.fill_step(g, rids, starts_a, n_tok, table, slots)
            parts += [slots, table]
        names: list[str] = []
        for provider in self._providers.values():
            for name, arr in provider.step_inputs(host).items():
                if name in names:
                    raise ValueError(f"two parts ask for a per-step array named {name!r}")
                names.append(name)
                parts.append(np.ascontiguousarray(arr, dtype=np.int32))
        # One buffer, one copy; every piece starts on a 16-byte boundary.
        offsets, total = [], 0
        for p in parts:
            offsets.append(total)
            total += (p.size + 3) & ~3
        return _Layout(parts, names, offsets, max(total, 4), host)

    def needed_width(self, entries: list[StepEntry], group: int) -> int:
        return self.needed_widths(entries)[group]

    def needed_widths(self, entries: list[StepEntry]) -> list[int]:
        """The block-table width that the step's requests need, per group."""
        rids = np.fromiter((e.request_id for e in entries), dtype=np.uint64, count=len(entries))
        return [max(1, int(w)) for w in self.cache.describe(rids)[1].max(axis=0)]

    def _context(self, lay: _Layout, dev: torch.Tensor):
        views = [dev[o:o + p.size].view(p.shape) for p, o in zip(lay.parts, lay.offsets)]
        ids_d, pos_d, cu_d, klen_d, slots_d, want_d = views[:N_FIXED]
        n_groups = len(self.pool.group_windows)
        groups = [GroupTables(slots=views[N_FIXED + 2 * g], block_table=views[N_FIXED + 1 + 2 * g], window=w)
                  for g, w in enumerate(self.pool.group_windows)]
        inputs = dict(zip(lay.names, views[N_FIXED + 2 * n_groups:]))
        ctx = StepContext(kernels=self.kernels, num_tokens=sum(lay.host.q_lens), num_seqs=len(lay.host.q_lens),
                          positions=pos_d, cu_q=cu_d, k_len=klen_d, state_slots=slots_d, groups=groups, host=lay.host,
                          inputs=inputs, workspace=self._get_workspace)
        return ids_d, ctx, want_d

    def build_context(self, entries: list[StepEntry]):
        """Host arrays of the step -> one upload -> (ids, context, wanted rows)."""
        lay = self._layout(entries)
        host = np.zeros(lay.total, dtype=np.int32)
        lay.pack(host)
        return self._context(lay, torch.from_numpy(host).to("cuda"))

    # ---------------------------------------------------------------- running
    def run(self, entries: list[StepEntry]) -> torch.Tensor:
        """The forward pass of a step whose pages are taken; logits [wanted, vocab] in the element type."""
        if self.graphs and all(len(e.tokens) == 1 and e.want == [0] for e in entries):
            return self._run_decode_graph(entries)
        return self._run_eager(entries)

    def _run_eager(self, entries: list[StepEntry]) -> torch.Tensor:
        self.graph_stats["eager"] += 1
        ids, ctx, want = self.build_context(entries)
        # What the parts announced, before the first of them runs: a part that asks twice in its forward then
        # gets the same buffer both times.
        self._get_workspace(self.workspace_needed(ctx.host))
        return self.model.forward(ids, ctx, self.pool.entries, want)

    def _run_decode_graph(self, entries: list[StepEntry]) -> torch.Tensor:
        if self._poisoned is not None:
            raise GraphError(f"graph replay is switched off after a failure: {self._poisoned}")
        P = self.pool.page_size
        widths = [width_bucket(w) for w in self.needed_widths(entries)]
        # A mixer with state of its own would have to be told which rows are padding: no padding then.
        rows = len(entries) if self.pool.has_state else row_bucket(len(entries))
        key = (rows, tuple(widths))
        cap = self._captured.get(key)
        if cap is None and key not in self._seen:
            # First sight of a signature: eagerly, which also warms up every kernel it uses.
            self._seen.add(key)
            return self._run_eager(entries)
        # Launch geometry is frozen in the graph: it must cover every length the tables can hold.
        cover = min(max(widths) * P, self.model.spec.max_positions)
        lay = self._layout(entries, widths, rows, bound=cover)
        try:
            if cap is None:
                cap = self._capture(key, lay)
            else:
                self._captured.move_to_end(key)
                cap.copied.synchronize()                       # the staging buffer is free again
                lay.pack(cap.staging.numpy())
                cap.meta.copy_(cap.staging, non_blocking=True)
            cap.copied.record()
            cap.graph.replay()
        except Exception as e:
            self._poisoned = f"{type(e).__name__}: {e}"
            self._captured.clear()
            raise GraphError(f"graph capture or replay failed ({self._poisoned}); no further step is replayed") from e
        self.graph_stats["replayed"] += 1
        return cap.logits[:len(entries)]

    def _capture(self, key: tuple, lay: _Layout) -> _Captured:
        while len(self._captured) >= self.max_graphs:
            self._captured.popitem(last=False)                 # the least recently replayed
            self.graph_stats["evicted"] += 1
        workspace = self._get_workspace(self.workspace_needed(lay.host))
        staging = torch.empty(lay.total, dtype=torch.int32, pin_memory=True)
        meta = torch.zeros(lay.total, dtype=torch.int32, device="cuda")
        lay.pack(staging.numpy())
        meta.copy_(staging, non_blocking=True)
        ids, ctx, want = self._context(lay, meta)
        torch.cuda.synchronize()
        if self._graph_pool is None:
            # One memory pool for all captures: they never replay at the same time, so the
            # intermediates of one may lie where another's lay; each keeps its own logits.
            self._graph_pool = torch.cuda.graph_pool_handle()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, pool=self._graph_pool):
            logits = self.model.forward(ids, ctx, self.pool.entries, want)
        cap = _Captured(graph, meta, staging, logits, torch.cuda.Event(), workspace)
        self._captured[key] = cap
        self.graph_stats["captured"] += 1
        return cap

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
