"""The engine behind the Python entry point.

``NativeEngine`` is the engine: plan -> forward -> sample -> commit in C++ (``csrc/engine``, built as
``libvosti_engine.so``), with the face ``add_request``, ``step``, ``generate``, ``has_unfinished``.  It serves
every model whose architecture and part kinds are registered in the library or in a plugin loaded into it
(``load_plugin``); ``native_support`` asks the library.  A model made of parts that exist in Python alone
runs through ``vosti_amd.engine.Engine``, the Python step function over the same kernels, cache manager and
scheduler; ``vosti_amd.engine.create_engine`` picks.  For the same requests and settings both produce the
same tokens and logits (tests/test_native_engine_gpu.py).
"""
from __future__ import annotations

import ctypes
import json
from ctypes import c_char_p, c_float, c_int, c_int64, c_uint64, c_void_p
from pathlib import Path

import numpy as np

from ..kernels import build
from ..kernels.ops import dtype_name
from ..sampling import SamplingParams

ABI_VERSION = 3
_LIB = None


class NativeEngineError(RuntimeError):
    pass


def _lib():
    global _LIB
    if _LIB is None:
        import torch  # noqa: F401  (one HIP runtime per process: torch's, loaded first)
        from ..cache.host import host_lib
        host_lib()        # linked against it: one cache manager, scheduler and registry of architectures per process
        # Global, so that a plugin loaded later finds the registries it registers with.
        lib = ctypes.CDLL(str(build.ensure("engine_lib")), mode=ctypes.RTLD_GLOBAL)
        lib.ve_abi_version.restype = c_int
        if lib.ve_abi_version() != ABI_VERSION:
            raise NativeEngineError(f"libvosti_engine.so has ABI {lib.ve_abi_version()}, expected {ABI_VERSION}; rebuild it")
        lib.ve_load_plugin.argtypes = [c_char_p, c_char_p, c_int]
        lib.ve_supports.argtypes = [c_char_p, c_char_p, c_int]
        lib.ve_create.restype = c_void_p
        lib.ve_create.argtypes = [c_char_p, c_char_p, c_char_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_uint64,
                                  c_char_p, c_int]
        lib.ve_destroy.argtypes = [c_void_p]
        lib.ve_add_request.restype = c_int64
        lib.ve_add_request.argtypes = [c_void_p, c_void_p, c_int, c_int, c_float, c_uint64, c_void_p, c_int, c_int, c_char_p, c_int]
        lib.ve_step.restype = c_int
        lib.ve_step.argtypes = [c_void_p, c_void_p, c_int, c_char_p, c_int]
        lib.ve_has_unfinished.argtypes = [c_void_p]
        lib.ve_synchronize.argtypes = [c_void_p, c_char_p, c_int]
        lib.ve_stats.argtypes = [c_void_p, c_void_p]
        lib.ve_cache_check.argtypes = [c_void_p, c_char_p, c_int]
        lib.ve_trace_add_request.argtypes = [c_void_p, c_int64, c_void_p, c_int, c_char_p, c_int]
        lib.ve_trace_step.restype = c_int64
        lib.ve_trace_step.argtypes = [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_char_p, c_int]
        lib.ve_trace_has_request.argtypes = [c_void_p, c_int64]
        lib.ve_trace_finish.argtypes = [c_void_p, c_int64, c_char_p, c_int]
        _LIB = lib
    return _LIB


def load_plugin(path: str | Path) -> None:
    """Loads a shared library that registers part kinds and architectures of its own with the native engine
    (compiled against csrc/engine/parts.h; it exports ``vosti_plugin_register``)."""
    err = ctypes.create_string_buffer(2048)
    if _lib().ve_load_plugin(str(path).encode(), err, len(err)) != 0:
        raise NativeEngineError(err.value.decode(errors="replace"))


def load_plugins_from_environment() -> None:
    """VOSTI_PLUGINS: paths of plugins, separated by colons, as the native program reads it."""
    import os
    for path in (os.environ.get("VOSTI_PLUGINS") or "").split(":"):
        if path:
            load_plugin(path)


def native_support(model_dir: str | Path) -> tuple[bool, str]:
    """Whether the native engine can run the model in ``model_dir``, and if not, why: (False, reason) when the
    architecture or one of its part kinds is registered only in Python.  A configuration that breaks a rule
    raises ``ConfigError`` with the library's text."""
    from ..config import ConfigError
    err = ctypes.create_string_buffer(2048)
    rc = _lib().ve_supports(str(model_dir).encode(), err, len(err))
    if rc < 0:
        raise ConfigError(err.value.decode(errors="replace"))
    return rc == 1, err.value.decode(errors="replace")


class NativeEngine:
    def __init__(self, model_dir: str | Path, *, dtype="bfloat16", num_pages: int = 32, page_size: int = 64, max_num_seqs: int = 8,
                 max_num_batched_tokens: int = 4096, enable_prefix_cache: bool = True, max_model_len: int | None = None,
                 graphs: bool = False, random_weights_seed: int | None = None):
        """The arguments of ``Engine``; ``model_dir`` must be a folder (config.json and safetensors).  With
        ``random_weights_seed`` the folder needs config.json only and the weights are drawn on the GPU from
        that seed (the values ``write_random_model`` stores for it)."""
        self._lib = _lib()
        name = dtype_name(dtype)
        kernels = build.ensure(name)              # the engine loads the kernel library of its precision from here
        self._err = ctypes.create_string_buffer(4096)
        self.max_num_seqs = max_num_seqs
        self._h = self._lib.ve_create(str(model_dir).encode(), str(kernels.parent).encode(), name.encode(), num_pages, page_size,
                                      max_num_seqs, max_num_batched_tokens, 1 if enable_prefix_cache else 0, max_model_len or 0,
                                      1 if graphs else 0, 0 if random_weights_seed is None else 1,
                                      (random_weights_seed or 0) & (2**64 - 1), self._err, len(self._err))
        if not self._h:
            raise NativeEngineError(self._err.value.decode(errors="replace"))
        self._out = np.empty((max_num_seqs + 1, 2), dtype=np.int64)
        self.steps = 0

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.ve_destroy(h)

    def _fail(self):
        raise NativeEngineError(self._err.value.decode(errors="replace"))

    # ------------------------------------------------------------- requests
    def add_request(self, prompt_ids: list[int], params: SamplingParams | None = None) -> int:
        params = params or SamplingParams()
        prompt = np.asarray(prompt_ids, dtype=np.int32)
        eos = np.asarray(params.eos_token_ids, dtype=np.int32)
        rid = self._lib.ve_add_request(self._h, prompt.ctypes.data, len(prompt), params.max_tokens, params.temperature,
                                       params.seed & (2**64 - 1), eos.ctypes.data if len(eos) else None, len(eos),
                                       1 if params.ignore_eos else 0, self._err, len(self._err))
        if rid < 0:
            raise ValueError(self._err.value.decode(errors="replace"))
        return rid

    def has_unfinished(self) -> bool:
        return bool(self._lib.ve_has_unfinished(self._h))

    # ----------------------------------------------------------------- step
    def step(self) -> dict[int, int]:
        """One engine step.  Returns {request id: emitted token} for the requests that emitted one."""
        n = self._lib.ve_step(self._h, self._out.ctypes.data, len(self._out), self._err, len(self._err))
        if n < 0:
            self._fail()
        self.steps += 1
        return {int(r): int(t) for r, t in self._out[:n]}

    def synchronize(self) -> None:
        if self._lib.ve_synchronize(self._h, self._err, len(self._err)) != 0:
            self._fail()

    def stats(self) -> dict:
        out = np.zeros(10, dtype=np.int64)
        self._lib.ve_stats(self._h, out.ctypes.data)
        names = ("eager", "captured", "replayed", "evicted")
        return {"graph_stats": dict(zip(names, map(int, out[:4]))), "prefix_hit_requests": int(out[4]), "prefix_hits": int(out[5]),
                "preemptions": int(out[6]), "cache_requests": int(out[7]), "vocab_size": int(out[8]), "max_positions": int(out[9])}

    def cache_check(self) -> str:
        buf = ctypes.create_string_buffer(1024)
        self._lib.ve_cache_check(self._h, buf, len(buf))
        return buf.value.decode()

    # --------------------------------------------------------------- replay
    # The step function alone (what bin/trace_run drives): given tokens in, logits out; no scheduler, no sampling.
    # An engine is used either this way or through add_request / step, not both.
    def trace_add_request(self, rid: int, prompt: list[int]) -> int:
        """Announces a request's whole prompt (prefix cache on); returns how many of its first tokens are cached."""
        p = np.asarray(prompt, dtype=np.int32)
        cached = self._lib.ve_trace_add_request(self._h, rid, p.ctypes.data, len(p), self._err, len(self._err))
        if cached < 0:
            self._fail()
        return cached

    def trace_step(self, entries: list[tuple[int, list[int], list[int]]]) -> np.ndarray:
        """entries: (request id, its next tokens, wanted places among them).  float32 logits [wanted, vocabulary]."""
        ids = np.asarray([e[0] for e in entries], dtype=np.int64)
        tok_off = np.cumsum([0] + [len(e[1]) for e in entries], dtype=np.int64).astype(np.int32)
        want_off = np.cumsum([0] + [len(e[2]) for e in entries], dtype=np.int64).astype(np.int32)
        tokens = np.asarray([t for e in entries for t in e[1]], dtype=np.int32)
        want = np.asarray([w for e in entries for w in e[2]], dtype=np.int32)
        vocab = self.stats()["vocab_size"]
        out = np.empty((int(want_off[-1]), vocab), dtype=np.float32)
        rows = self._lib.ve_trace_step(self._h, len(entries), ids.ctypes.data, tok_off.ctypes.data, tokens.ctypes.data,
                                       want_off.ctypes.data, want.ctypes.data, out.ctypes.data, out.size, self._err, len(self._err))
        if rows < 0:
            self._fail()
        return out[:rows]

    def trace_has_request(self, rid: int) -> bool:
        return bool(self._lib.ve_trace_has_request(self._h, rid))

    def trace_finish(self, rid: int) -> None:
        if self._lib.ve_trace_finish(self._h, rid, self._err, len(self._err)) != 0:
            self._fail()

    # ------------------------------------------------------------- generate
    def generate(self, prompts: list[list[int]], params: SamplingParams | list[SamplingParams] | None = None,
                 arrival_steps: list[int] | None = None, trace=None) -> list[list[int]]:
        """As ``Engine.generate``: ``arrival_steps[i]`` delays prompt i until that engine step; ``trace`` gets one
        JSON line per step (without the ids scheduled, which stay inside the native engine)."""
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
                trace.write(json.dumps({"step": step, "arrived": arrived,
                                        "emitted": {str(ids.get(r, r)): t for r, t in emitted.items()}}) + "\n")
            step += 1
        return outputs
