"""Python face of the plain C++ references of the kernels (csrc/host/reference.cpp).

Host code on numpy arrays of float32; ``bf16=True`` rounds what the kernels store in the element type.
They are what the kernels are checked against, beside the plain Python implementation under tests/;
nothing on the path from tokens to logits calls them.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_void_p

import numpy as np

from ..cache.host import host_lib

_READY = False


def _lib():
    global _READY
    lib = host_lib()
    if not _READY:
        P, I, F = c_void_p, c_int, c_float
        sigs = {
            "vh_ref_embedding": (None, P, P, P, I, I),
            "vh_ref_rmsnorm": (None, P, P, P, I, I, F, I),
            "vh_ref_add_rmsnorm": (None, P, P, P, P, I, I, F, I),
            "vh_ref_gemm": (None, P, P, P, I, I, I, I),
            "vh_ref_swiglu": (None, P, P, I, I, I),
            "vh_ref_qkv_post": (None, P, P, P, P, P, P, P, P, I, P, P, I, I, I, I, I, F, I),
            "vh_ref_paged_attention": (None, P, P, P, P, P, I, P, P, I, I, I, I, I, I, F, I),
            "vh_ref_argmax": (I, P, I),
            "vh_ref_sample": (I, P, I, F, F),
            "vh_ref_round_bf16": (F, F),
        }
        for name, (res, *args) in sigs.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, list(args)
        _READY = True
    return lib


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _i32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.int32)


def _p(a):
    return None if a is None else a.ctypes.data


def embedding(table, ids) -> np.ndarray:
    table, ids = _f32(table), _i32(ids)
    out = np.empty((ids.shape[0], table.shape[1]), dtype=np.float32)
    _lib().vh_ref_embedding(_p(out), _p(table), _p(ids), ids.shape[0], table.shape[1])
    return out


def rmsnorm(x, w, eps: float, bf16: bool) -> np.ndarray:
    x, w = _f32(x), _f32(w)
    H = x.shape[-1]
    out = np.empty_like(x)
    _lib().vh_ref_rmsnorm(_p(out), _p(x), _p(w), x.size // H, H, eps, int(bf16))
    return out


def add_rmsnorm(x, residual, w, eps: float, bf16: bool) -> tuple[np.ndarray, np.ndarray]:
    """Returns (normed, new residual)."""
    x, w = _f32(x), _f32(w)
    res = _f32(residual).copy()
    out = np.empty_like(x)
    _lib().vh_ref_add_rmsnorm(_p(out), _p(res), _p(x), _p(w), x.shape[0], x.shape[1], eps, int(bf16))
    return out, res


def gemm(act, w, bf16: bool) -> np.ndarray:
    act, w = _f32(act), _f32(w)
    out = np.empty((act.shape[0], w.shape[0]), dtype=np.float32)
    _lib().vh_ref_gemm(_p(out), _p(act), _p(w), act.shape[0], w.shape[0], act.shape[1], int(bf16))
    return out


def swiglu(gate_up, bf16: bool) -> np.ndarray:
    gu = _f32(gate_up)
    out = np.empty((gu.shape[0], gu.shape[1] // 2), dtype=np.float32)
    _lib().vh_ref_swiglu(_p(out), _p(gu), gu.shape[0], gu.shape[1] // 2, int(bf16))
    return out


def qkv_post(qkv, *, nq: int, nkv: int, d: int, k_cache, v_cache, page_size: int, q_w, k_w, eps: float, cos, sin,
             positions, slots, bf16: bool) -> np.ndarray:
    """Returns q [T, nq, d]; k_cache [pages, nkv, P, d] and v_cache [pages, nkv, d, P] (float32 arrays) are written in place."""
    qkv = _f32(qkv)
    T = qkv.shape[0]
    q_out = np.zeros((T, nq, d), dtype=np.float32)
    q_w = None if q_w is None else _f32(q_w)
    k_w = None if k_w is None else _f32(k_w)
    cos = None if cos is None else _f32(cos)
    sin = None if sin is None else _f32(sin)
    positions = None if positions is None else _i32(positions)
    slots = None if slots is None else _i32(slots)
    for c in (k_cache, v_cache):
        assert c is None or (c.dtype == np.float32 and c.flags.c_contiguous)
    _lib().vh_ref_qkv_post(_p(q_out), _p(k_cache), _p(v_cache), _p(qkv), _p(q_w), _p(k_w), _p(cos), _p(sin),
                           0 if cos is None else cos.shape[1], _p(positions), _p(slots), T, nq, nkv, d, page_size, eps, int(bf16))
    return q_out


def paged_attention(q, k_cache, v_cache, block_table, cu_q, k_len, *, scale: float, window: int = 0, bf16: bool) -> np.ndarray:
    q, kc, vc = _f32(q), _f32(k_cache), _f32(v_cache)
    bt, cu, kl = _i32(block_table), _i32(cu_q), _i32(k_len)
    T, nq, d = q.shape
    nkv, P = kc.shape[1], kc.shape[2]
    out = np.zeros_like(q)
    _lib().vh_ref_paged_attention(_p(out), _p(q), _p(kc), _p(vc), _p(bt), bt.shape[1], _p(cu), _p(kl), kl.shape[0], nq, nkv,
                                  d, P, window, scale, int(bf16))
    return out


def argmax(row) -> int:
    row = _f32(row)
    return _lib().vh_ref_argmax(_p(row), row.shape[0])


def sample(row, temperature: float, uniform: float) -> int:
    row = _f32(row)
    return _lib().vh_ref_sample(_p(row), row.shape[0], temperature, uniform)


def round_bf16(x: float) -> float:
    return float(_lib().vh_ref_round_bf16(x))
