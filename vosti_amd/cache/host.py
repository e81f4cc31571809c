"""Loads the native host library: the cache manager, the scheduler, the architectures' reading of config.json
and the rules that the native engine and this package share (rotation frequencies, the sizes that decode
steps are recorded with)."""
from __future__ import annotations

import ctypes
from ctypes import POINTER, c_char_p, c_double, c_int, c_int32, c_int64, c_uint64, c_void_p

from ..kernels import build

ABI_VERSION = 8
_LIB = None


def host_lib():
    global _LIB
    if _LIB is not None:
        return _LIB
    lib = ctypes.CDLL(str(build.ensure("host")), mode=ctypes.RTLD_GLOBAL)     # global: plugins of the native engine register with it
    lib.vh_abi_version.restype = c_int
    if lib.vh_abi_version() != ABI_VERSION:
        raise RuntimeError("libvosti_host.so is stale; rebuild it")
    I, U, P = c_int, c_uint64, c_void_p
    PI = POINTER(c_int32)

    def sig(name, restype, *args):
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = restype, list(args)

    sig("vh_cache_create", P, I, I, POINTER(c_int), POINTER(c_int), I, I)
    sig("vh_cache_destroy", None, P)
    sig("vh_cache_add_request", I, P, U, PI, I, POINTER(c_int))
    sig("vh_cache_reserve", I, P, U, I)
    sig("vh_cache_extend", I, P, U, PI, I)
    for n in ("commit", "abort_step", "finish", "has_request", "length", "pending", "state_slot"):
        sig(f"vh_cache_{n}", I, P, U)
    sig("vh_cache_num_logical_pages", I, P, U, I)
    sig("vh_cache_available_pages", I, P, I)
    sig("vh_cache_free_pages", I, P, I)
    for n in ("free_slots", "num_requests", "cached_blocks", "drop_cached"):
        sig(f"vh_cache_{n}", I, P)
    sig("vh_cache_prefix_hits", c_int64, P)
    sig("vh_cache_prefix_hit_requests", c_int64, P)
    sig("vh_cache_evictions", c_int64, P)
    sig("vh_cache_fill_block_table", I, P, U, I, c_void_p, I)
    sig("vh_cache_fill_slots", I, P, U, I, I, I, c_void_p)
    sig("vh_cache_check", I, P, c_char_p, I)
    sig("vh_cache_describe", I, P, I, c_void_p, c_void_p, c_void_p)
    sig("vh_cache_fill_step", I, P, I, I, c_void_p, c_void_p, c_void_p, I, I, c_void_p, I, c_void_p)
    sig("vh_sched_create", P, P, I, I, I)
    sig("vh_sched_destroy", None, P)
    sig("vh_sched_add_request", I, P, U, PI, I, I, PI, I, I)
    sig("vh_sched_plan", I, P, POINTER(c_int), POINTER(c_int))
    sig("vh_sched_get_plan", None, P, c_void_p, c_void_p)
    sig("vh_sched_commit", I, P, PI, I)
    sig("vh_sched_get_emitted", None, P, c_void_p)
    sig("vh_sched_abort_step", None, P)
    sig("vh_sched_num_planned_samples", I, P)
    sig("vh_sched_abort", I, P, U)
    sig("vh_sched_num_waiting", I, P)
    sig("vh_sched_num_running", I, P)
    sig("vh_sched_preemptions", c_int64, P)
    sig("vh_sched_is_live", I, P, U)
    sig("vh_describe_config", I, c_char_p, c_char_p, I, c_char_p, I)
    sig("vh_model_types", I, c_char_p, I)
    sig("vh_rotary_inverse_frequencies", None, c_double, I, c_void_p)
    sig("vh_graph_row_bucket", I, I)
    sig("vh_graph_width_bucket", I, I)
    sig("vh_max_graphs", I)
    _LIB = lib
    return lib


class UnknownArchitecture(ValueError):
    pass


def describe_config(raw: dict) -> dict:
    """What the native library's architecture makes of a config.json: the model's description as data
    (``model_spec_json`` in csrc/host/spec.h) with the typed configuration under "config".  ValueError with the
    library's text for a configuration that breaks a rule, UnknownArchitecture if the library has no such
    architecture."""
    import json
    lib = host_lib()
    text = json.dumps(raw).encode()
    err = ctypes.create_string_buffer(2048)
    cap = 1 << 16
    while True:
        out = ctypes.create_string_buffer(cap)
        n = lib.vh_describe_config(text, out, cap, err, len(err))
        if n == -2:
            raise UnknownArchitecture(err.value.decode(errors="replace"))
        if n < 0:
            raise ValueError(err.value.decode(errors="replace"))
        if n < cap:
            return json.loads(out.value.decode())
        cap = n + 1


def native_model_types() -> dict[str, str]:
    """model_type -> architecture name of every architecture the native library has."""
    lib = host_lib()
    out = ctypes.create_string_buffer(4096)
    lib.vh_model_types(out, len(out))
    return dict(line.split("=", 1) for line in out.value.decode().splitlines() if line)


def rotary_inverse_frequencies(theta: float, rotary_dim: int):
    """float32 numpy array [rotary_dim / 2]: 1 / theta^(2j / rotary_dim), the one routine every host uses."""
    import numpy as np
    out = np.empty(rotary_dim // 2, dtype=np.float32)
    host_lib().vh_rotary_inverse_frequencies(float(theta), int(rotary_dim), out.ctypes.data)
    return out


def graph_row_bucket(rows: int) -> int:
    return host_lib().vh_graph_row_bucket(int(rows))


def graph_width_bucket(pages: int) -> int:
    return host_lib().vh_graph_width_bucket(int(pages))


def max_graphs() -> int:
    return host_lib().vh_max_graphs()


def i32_array(values):
    arr = (c_int32 * len(values))(*values)
    return arr
