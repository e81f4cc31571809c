"""The engine: requests in, tokens out.

One step is plan -> forward -> sample -> commit, as in the reference
(src/exec/engine.rs:2795, 2862, 3258, 3427; docs/architecture.md:99-109).  The
scheduler decides the rows and takes their pages, the step function runs them
and returns logits at the rows that end a request's tokens, the sampler draws
one token per such row on the GPU, and one readback per step brings the tokens
to the host, where the scheduler appends them and retires finished requests.
"""
from __future__ import annotations

import json
from pathlib import Path

import numpy as np
import torch

from ..cache import CachePool
from ..models import DecoderModel, load_model
from ..sampling import SamplingParams, uniform_for
from .observe import LogitsObserver
from .scheduler import Scheduler
from .step import ModelRunner, StepEntry


class Engine:
    def __init__(self, model: DecoderModel | str | Path, *, dtype="bfloat16", num_pages: int = 32, page_size: int = 64,
                 max_num_seqs: int = 8, max_num_batched_tokens: int = 4096, enable_prefix_cache: bool = True,
                 max_model_len: int | None = None, graphs: bool = False):
        """``num_pages`` is the reference's VOSTI_NUM_BLOCKS (default 32 pages of 64 tokens),
        ``max_num_seqs`` VOSTI_MAX_SEQS and ``max_num_batched_tokens`` VOSTI_MAX_BATCHED_TOKENS
        (examples/support/engine_setup.rs:57-69); ``graphs`` is VOSTI_CUDA_GRAPH: steps of decoded tokens
        only are replayed from captured HIP graphs (engine_setup.rs:79-81)."""
        self.model = load_model(model, dtype) if isinstance(model, (str, Path)) else model
        self.kernels = self.model.kernels
        # One state slot per request that can be alive: those running plus the one being admitted.
        self.pool = CachePool(self.model, page_size=page_size, num_pages=num_pages, num_slots=max_num_seqs + 1,
                              prefix_cache=enable_prefix_cache)
        self.runner = ModelRunner(self.model, self.pool, graphs=graphs)
        self.cache = self.pool.manager
        self.max_model_len = min(max_model_len or self.model.spec.max_positions, self.model.spec.max_positions)
        self.scheduler = Scheduler(self.cache, max_num_seqs, max_num_batched_tokens, self.max_model_len)
        # Fixed-size per-request state, by state slot: the sampler's.
        n = max_num_seqs + 1
        self.slot_temperature = np.zeros(n, dtype=np.float32)
        self.slot_seed = np.zeros(n, dtype=np.uint64)
        self.slot_owner = np.full(n, -1, dtype=np.int64)      # the request whose state the slot holds
        self._params: dict[int, SamplingParams] = {}
        self._next_id = 0
        self.steps = 0
        self.last_scheduled: list[int] = []
        # VOSTI_LOGITS_DIGEST / VOSTI_LOGITS_OBSERVER_DIR: hashes or copies of every sampled logits row, to
        # compare runs that batch differently (python/vosti_kernels/kernels.py:1020-1033).
        self.observer = LogitsObserver()

    # ------------------------------------------------------------- requests
    def add_request(self, prompt_ids: list[int], params: SamplingParams | None = None, request_id: int | None = None) -> int:
        params = params or SamplingParams()
        if request_id is None:
            request_id = self._next_id
        self._next_id = max(self._next_id, request_id + 1)
        vocab = self.model.spec.vocab_size
        if any((not isinstance(t, int)) or t < 0 or t >= vocab for t in prompt_ids):
            raise ValueError(f"prompt token outside [0, {vocab})")
        # A request without end tokens runs to max_tokens.
        status = self.scheduler.add_request(request_id, list(prompt_ids), params.max_tokens, params.eos_token_ids,
                                            params.ignore_eos or not params.eos_token_ids)
        if status != "Accepted":
            raise ValueError(f"request {request_id} refused: {status}")
        self._params[request_id] = params
        return request_id

    def has_unfinished(self) -> bool:
        return bool(self._params)

    # ----------------------------------------------------------------- step
    def step(self) -> dict[int, int]:
        """One engine step.  Returns {request id: emitted token} for the requests that emitted one."""
        rows = self.scheduler.plan()
        self.last_scheduled = [r.request_id for r in rows]
        if not rows:
            return {}
        try:
            sampled = self._forward_and_sample(rows)
        except BaseException:
            # Nothing of the step counts: the rows' tokens stay uncomputed, their pages stay with their
            # requests, and the next plan() decides again.
            self.scheduler.abort_step()
            raise
        emitted = self.scheduler.commit(sampled)
        self.steps += 1
        out = {}
        for e in emitted:
            out[e.request_id] = e.token
            if e.finished:
                self._params.pop(e.request_id, None)
        return out

    def _forward_and_sample(self, rows) -> list[int]:
        """Runs the planned rows and draws one token per sampled row (one readback)."""
        entries = [StepEntry(r.request_id, r.tokens, [len(r.tokens) - 1] if r.sample else []) for r in rows]
        sampling = [r for r in rows if r.sample]
        logits = self.runner.run(entries)
        sampled: list[int] = []
        if sampling and self.observer.active:
            self.observer.rows(self.kernels.to_f32(logits).cpu().numpy(), [rows.index(r) for r in sampling], self.steps,
                               str(self.kernels.dtype).replace("torch.", ""))
        if sampling:
            temps = np.zeros(len(sampling), dtype=np.float32)
            unis = np.zeros(len(sampling), dtype=np.float32)
            for i, r in enumerate(sampling):
                # The slot holds the request's sampler state.  A request gets its slot at admission, inside
                # plan(), so the state is written when the request's first sampled row shows up in it.
                if self.slot_owner[r.state_slot] != r.request_id:
                    p = self._params[r.request_id]
                    self.slot_owner[r.state_slot] = r.request_id
                    self.slot_temperature[r.state_slot] = p.temperature
                    self.slot_seed[r.state_slot] = p.seed & ((1 << 64) - 1)
                temps[i] = self.slot_temperature[r.state_slot]
                unis[i] = uniform_for(int(self.slot_seed[r.state_slot]), r.output_index)
            if (temps > 0).any():
                both = torch.from_numpy(np.stack([temps, unis])).to("cuda")
                ids = self.kernels.sample(logits, both[0], both[1])
            else:
                ids = self.kernels.sample(logits)
            sampled = ids.cpu().tolist()     # the step's one synchronisation
        return sampled

    # ------------------------------------------------------------- generate
    def generate(self, prompts: list[list[int]], params: SamplingParams | list[SamplingParams] | None = None,
                 arrival_steps: list[int] | None = None, trace=None) -> list[list[int]]:
        """Generates for every prompt; ``arrival_steps[i]`` delays prompt i until that engine step
        (the reference's prepared-request TSV has the same column: examples/support/engine_benchmark.rs:89-165).
        ``trace``: a text file that gets one JSON line per step with the requests that arrived, the ids
        scheduled and the tokens emitted (engine_benchmark.rs:212-220, 273-317)."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        arrival_steps = arrival_steps or [0] * len(prompts)
        pending = sorted(range(len(prompts)), key=lambda i: (arrival_steps[i], i))
        ids: dict[int, int] = {}
        outputs: list[list[int]] = [[] for _ in prompts]
        step = 0
        while pending or self.has_unfinished():
            arrived = []
            while pending and arrival_steps[pending[0]] <= step:
                i = pending.pop(0)
                ids[self.add_request(prompts[i], params[i])] = i
                arrived.append(i)
            emitted = self.step()
            for rid, tok in emitted.items():
                if rid in ids:
                    outputs[ids[rid]].append(tok)
            if trace is not None:
                trace.write(json.dumps({"step": step, "arrived": arrived, "scheduled": self.last_scheduled,
                                        "emitted": {str(ids.get(r, r)): t for r, t in emitted.items()},
                                        "cached_prefix_pages": self.cache.prefix_hits()}) + "\n")
            step += 1
        return outputs
