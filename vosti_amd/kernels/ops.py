"""Python bindings of the gfx950 kernel libraries.

``kernels_for(dtype)`` returns a ``Kernels`` object bound to the library built
for that element type.  Every method checks operand shapes, types and devices
on the host before a launch, because a kernel that reads out of bounds can take
the GPU down; there is no CPU path, and a missing or stale library is an error.
All launches go to torch's current stream.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_int64, c_uint64, c_void_p

import torch

from . import build

ABI_VERSION = 13
SEGMENT_KEYS = 256
ATTN_ITEM_ROWS = 128      # rows of one prompt item of paged_attention

_DTYPES = {"bf16": torch.bfloat16, "f32": torch.float32}
_NAMES = {torch.bfloat16: "bf16", torch.float32: "f32", "bfloat16": "bf16", "float32": "f32", "bf16": "bf16",
          "f32": "f32", "fp32": "f32"}


class KernelError(RuntimeError):
    pass


def dtype_name(dtype) -> str:
    try:
        return _NAMES[dtype]
    except KeyError:
        raise ValueError(f"unsupported element type {dtype!r}; use bfloat16 or float32") from None


def _sig(fn, *argtypes):
    fn.argtypes = list(argtypes)
    fn.restype = c_int
    return fn


class Kernels:
    def __init__(self, name: str):
        self.name = name
        self.dtype = _DTYPES[name]
        path = build.ensure(name)
        self.path = str(path)
        lib = ctypes.CDLL(self.path)
        lib.vk_last_error.restype = ctypes.c_char_p
        lib.vk_abi_version.restype = c_int
        lib.vk_elem_bytes.restype = c_int
        if lib.vk_abi_version() != ABI_VERSION:
            raise KernelError(f"{path} has ABI {lib.vk_abi_version()}, expected {ABI_VERSION}; rebuild it")
        if lib.vk_elem_bytes() != torch.empty((), dtype=self.dtype).element_size():
            raise KernelError(f"{path} was built for another element type")
        P, I, L, F = c_void_p, c_int, c_int64, c_float
        _sig(lib.vk_embedding, P, P, P, I, I, I, P)
        _sig(lib.vk_rmsnorm, P, P, P, I, I, I, I, L, L, F, P)
        _sig(lib.vk_add_rmsnorm, P, P, P, P, I, I, I, F, P)
        _sig(lib.vk_swiglu, P, P, I, I, P)
        _sig(lib.vk_gather_rows, P, P, P, I, I, P)
        _sig(lib.vk_cast_to_f32, P, P, L, P)
        _sig(lib.vk_cast_from_f32, P, P, L, P)
        _sig(lib.vk_rope_tables, P, P, P, I, I, P)
        _sig(lib.vk_fill_random, P, L, c_uint64, I, F, F, P)
        _sig(lib.vk_pull, P, L, P, P)
        _sig(lib.vk_gemm, P, P, P, I, I, I, L, L, I, P)
        _sig(lib.vk_gemm_swiglu, P, P, P, I, I, I, L, L, P)
        _sig(lib.vk_gemm_swiglu_supported, I, I, I)
        _sig(lib.vk_gemm_split, P, P, P, I, I, I, L, L, I, P, L, P)
        lib.vk_gemm_split_floats.argtypes = [I, I, I, I]
        lib.vk_gemm_split_floats.restype = c_int64
        _sig(lib.vk_gemm_split_preferred, I, I, I, I)
        _sig(lib.vk_qkv_post, P, L, P, P, P, P, P, I, P, P, I, P, P, I, I, I, I, I, F, P)
        _sig(lib.vk_paged_attention, P, P, P, P, P, I, P, P, P, I, I, I, P, I, I, I, I, I, I, F, P)
        _sig(lib.vk_sample, P, P, P, P, P, I, I, L, P)
        lib.vk_sample_scratch_words.argtypes = [I]
        lib.vk_sample_scratch_words.restype = c_int
        lib.vk_attn_scratch_floats.argtypes = [I, I, I, I]
        lib.vk_attn_scratch_floats.restype = c_int64
        lib.vk_attn_segment_keys.restype = c_int
        assert lib.vk_attn_segment_keys() == SEGMENT_KEYS
        lib.vk_attn_item_rows.restype = c_int
        assert lib.vk_attn_item_rows() == ATTN_ITEM_ROWS
        self.lib = lib

    # ------------------------------------------------------------ helpers
    def _call(self, fn, *args):
        if fn(*args) != 0:
            raise KernelError(self.lib.vk_last_error().decode())

    @staticmethod
    def _stream() -> int:
        return torch.cuda.current_stream().cuda_stream

    def _elem(self, t: torch.Tensor, what: str, *shape) -> int:
        self._check(t, what, self.dtype, shape)
        return t.data_ptr()

    @staticmethod
    def _check(t: torch.Tensor, what: str, dtype, shape=()) -> None:
        if not isinstance(t, torch.Tensor):
            raise KernelError(f"{what} is not a tensor")
        if not t.is_cuda:
            raise KernelError(f"{what} is not on the GPU")
        if t.dtype != dtype:
            raise KernelError(f"{what} has type {t.dtype}, expected {dtype}")
        if not t.is_contiguous():
            raise KernelError(f"{what} is not contiguous")
        if shape and tuple(t.shape) != tuple(shape):
            raise KernelError(f"{what} has shape {tuple(t.shape)}, expected {tuple(shape)}")

    def _i32(self, t: torch.Tensor, what: str, *shape) -> int:
        self._check(t, what, torch.int32, shape)
        return t.data_ptr()

    def _f32(self, t: torch.Tensor, what: str, *shape) -> int:
        self._check(t, what, torch.float32, shape)
        return t.data_ptr()

    def _weight(self, w: torch.Tensor, what: str, n: int) -> tuple[int, int]:
        """A norm weight may be stored as elements or as float."""
        if w.dtype == torch.float32 and self.dtype != torch.float32:
            self._check(w, what, torch.float32, (n,))
            return w.data_ptr(), 1
        self._check(w, what, self.dtype, (n,))
        return w.data_ptr(), 1 if self.dtype == torch.float32 else 0

    def empty(self, *shape) -> torch.Tensor:
        return torch.empty(shape, dtype=self.dtype, device="cuda")

    # ---------------------------------------------------------------- ops
    def embedding(self, table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        """out[t] = table[ids[t]].  ids (int32, on the GPU) must lie in [0, V): the caller checks on the host."""
        V, H = table.shape
        T = ids.shape[0]
        out = self.empty(T, H) if out is None else out
        self._call(self.lib.vk_embedding, self._elem(out, "out", T, H), self._elem(table, "table", V, H),
                   self._i32(ids, "ids", T), T, H, V, self._stream())
        return out

    def rmsnorm(self, x: torch.Tensor, w: torch.Tensor, eps: float, out: torch.Tensor | None = None) -> torch.Tensor:
        """Row-wise RMSNorm over the last axis of a contiguous tensor."""
        H = x.shape[-1]
        rows = x.numel() // H
        out = torch.empty_like(x) if out is None else out
        wp, wf = self._weight(w, "norm weight", H)
        self._call(self.lib.vk_rmsnorm, self._elem(out, "out", *x.shape), self._elem(x, "x"), wp, wf, rows, H, 1, H, H,
                   float(eps), self._stream())
        return out

    def add_rmsnorm(self, x: torch.Tensor, residual: torch.Tensor, w: torch.Tensor, eps: float,
                    out: torch.Tensor | None = None) -> torch.Tensor:
        """residual += x in place (fp32 sum, stored rounded); returns rmsnorm of the unrounded sum."""
        T, H = x.shape
        out = torch.empty_like(x) if out is None else out
        wp, wf = self._weight(w, "norm weight", H)
        self._call(self.lib.vk_add_rmsnorm, self._elem(out, "out", T, H), self._elem(residual, "residual", T, H),
                   self._elem(x, "x", T, H), wp, wf, T, H, float(eps), self._stream())
        return out

    def swiglu(self, gate_up: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        T, I2 = gate_up.shape
        if I2 % 2:
            raise KernelError(f"swiglu: width {I2} of the gate/up tensor is odd")
        I = I2 // 2
        out = self.empty(T, I) if out is None else out
        self._call(self.lib.vk_swiglu, self._elem(out, "out", T, I), self._elem(gate_up, "gate_up", T, I2), T, I,
                   self._stream())
        return out

    def gather_rows(self, x: torch.Tensor, rows: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        """out[r] = x[rows[r]].  rows (int32, on the GPU) must lie in [0, T): the caller checks on the host."""
        T, H = x.shape
        R = rows.shape[0]
        out = self.empty(R, H) if out is None else out
        self._call(self.lib.vk_gather_rows, self._elem(out, "out", R, H), self._elem(x, "x", T, H),
                   self._i32(rows, "rows", R), R, H, self._stream())
        return out

    def to_f32(self, x: torch.Tensor) -> torch.Tensor:
        out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
        self._call(self.lib.vk_cast_to_f32, self._f32(out, "out"), self._elem(x, "x"), x.numel(), self._stream())
        return out

    def from_f32(self, x: torch.Tensor) -> torch.Tensor:
        out = torch.empty(x.shape, dtype=self.dtype, device=x.device)
        self._call(self.lib.vk_cast_from_f32, self._elem(out, "out"), self._f32(x, "x"), x.numel(), self._stream())
        return out

    def rope_tables(self, inv_freq: torch.Tensor, max_pos: int) -> tuple[torch.Tensor, torch.Tensor]:
        half = inv_freq.shape[0]
        cos, sin = self.empty(max_pos, half), self.empty(max_pos, half)
        self._call(self.lib.vk_rope_tables, cos.data_ptr(), sin.data_ptr(), self._f32(inv_freq, "inv_freq", half),
                   max_pos, half, self._stream())
        return cos, sin

    def pull(self, t: torch.Tensor, sink: torch.Tensor) -> None:
        """Reads ``t`` (contiguous) once and keeps nothing: the yardstick of what a kernel that must read it can
        reach.  ``sink``: an int32 tensor on the GPU that is practically never written."""
        if not t.is_contiguous() or not t.is_cuda:
            raise KernelError("pull: a contiguous tensor on the GPU is needed")
        self._call(self.lib.vk_pull, t.data_ptr(), t.numel() * t.element_size(), self._i32(sink, "sink"), self._stream())

    def fill_random(self, out: torch.Tensor, seed: int, kind: int, p0: float, p1: float) -> None:
        self._call(self.lib.vk_fill_random, self._elem(out, "out"), out.numel(), c_uint64(seed & (2**64 - 1)), kind,
                   float(p0), float(p1), self._stream())

    def gemm_workspace_floats(self, M: int, rows: int, K: int, swiglu: bool = False, force: bool = False) -> int:
        """float32 elements of workspace with which ``gemm`` / ``gemm_swiglu`` take the route through chunk
        sums for these sizes, or 0 where that route does not exist or is the slower one (``force``: where it
        does not exist).  A part adds this to what it asks of the step's workspace."""
        if not force and not self.lib.vk_gemm_split_preferred(M, rows, K, 1 if swiglu else 0):
            return 0
        return int(self.lib.vk_gemm_split_floats(M, rows, K, 1 if swiglu else 0))

    def _split(self, out, act, w, M, rows, K, lda, ldo, swiglu, workspace, force=False) -> bool:
        """Runs the product through chunk sums in ``workspace`` if that is the faster route and it fits."""
        if workspace is None:
            if force:
                raise KernelError("gemm: the route through chunk sums needs a workspace")
            return False
        need = self.gemm_workspace_floats(M, rows, K, swiglu, force)
        if need == 0 or workspace.numel() < need:
            if force:
                raise KernelError(f"gemm: no route through chunk sums for M={M} rows={rows} K={K}, or the workspace "
                                  f"of {workspace.numel()} floats is smaller than {need}")
            return False
        self._call(self.lib.vk_gemm_split, out.data_ptr(), act.data_ptr(), w.data_ptr(), M, rows, K, lda, ldo,
                   1 if swiglu else 0, self._f32(workspace, "workspace"), workspace.numel(), self._stream())
        return True

    def gemm(self, act: torch.Tensor, w: torch.Tensor, out: torch.Tensor | None = None, kernel: int = 0,
             workspace: torch.Tensor | None = None) -> torch.Tensor:
        """out = act @ w.T with w in [out_features, in_features] layout.

        ``act`` may be a view of rows with a row stride (its last axis contiguous).  ``workspace``: float32
        scratch; with enough of it (``gemm_workspace_floats``) some sizes take a faster route to the same
        bits.  ``kernel`` 14 forces that route (tests)."""
        M, K = act.shape
        N, K2 = w.shape
        if K2 != K:
            raise KernelError(f"gemm: activation width {K} differs from the weight's input width {K2}")
        self._check(w, "weight", self.dtype, (N, K))
        if not act.is_cuda or act.dtype != self.dtype or act.stride(1) != 1:
            raise KernelError("gemm: activation must be a GPU tensor of the element type with a contiguous last axis")
        lda = act.stride(0) if M > 1 else max(K, act.stride(0))
        out = self.empty(M, N) if out is None else out
        self._elem(out, "out", M, N)
        if kernel in (0, 14) and self._split(out, act, w, M, N, K, lda, N, False, workspace, force=kernel == 14):
            return out
        self._call(self.lib.vk_gemm, out.data_ptr(), act.data_ptr(), w.data_ptr(), M, N, K, lda, N, kernel,
                   self._stream())
        return out

    def gemm_swiglu(self, act: torch.Tensor, w_gate_up: torch.Tensor, workspace: torch.Tensor | None = None,
                    split: bool = False) -> torch.Tensor:
        """silu(act @ w_gate.T) * (act @ w_up.T) with w_gate_up = [gate rows; up rows].

        One launch where the sizes allow it, else the projection and the activation one after the
        other; the result is the same bits either way.  ``split`` forces the route through chunk sums in
        ``workspace`` (tests)."""
        M, K = act.shape
        N2, K2 = w_gate_up.shape
        if K2 != K or N2 % 2:
            raise KernelError(f"gemm_swiglu: activation [{M}, {K}] does not fit a gate/up weight [{N2}, {K2}]")
        I = N2 // 2
        if not (act.is_contiguous() and self.lib.vk_gemm_swiglu_supported(M, I, K)):
            return self.swiglu(self.gemm(act, w_gate_up, workspace=workspace))
        self._elem(act, "activation", M, K)
        self._elem(w_gate_up, "weight", N2, K)
        out = self.empty(M, I)
        if self._split(out, act, w_gate_up, M, N2, K, K, I, True, workspace, force=split):
            return out
        self._call(self.lib.vk_gemm_swiglu, out.data_ptr(), act.data_ptr(), w_gate_up.data_ptr(), M, I, K, K, I,
                   self._stream())
        return out

    def qkv_post(self, qkv: torch.Tensor, *, nq: int, nkv: int, d: int, q_out: torch.Tensor | None,
                 k_cache: torch.Tensor | None, v_cache: torch.Tensor | None, page_size: int,
                 q_w: torch.Tensor | None, k_w: torch.Tensor | None, eps: float,
                 cos: torch.Tensor | None, sin: torch.Tensor | None, positions: torch.Tensor | None,
                 slots: torch.Tensor | None) -> torch.Tensor | None:
        """Head norm, rotation and cache store of a [T, (nq + 2 nkv) d] row tensor (see qkv_post.hip).

        Positions must be below the tables' row count and slots inside the caches: checked by the caller on the host."""
        T, W = qkv.shape
        if W != (nq + 2 * nkv) * d:
            raise KernelError(f"qkv_post: row width {W} is not (nq + 2 nkv) * d = {(nq + 2 * nkv) * d}")
        self._elem(qkv, "qkv", T, W)
        if nq:
            q_out = self.empty(T, nq, d) if q_out is None else q_out
            self._elem(q_out, "q_out", T, nq, d)
        wf = 0
        qwp = kwp = None
        if q_w is not None:
            qwp, wf = self._weight(q_w, "q norm weight", d)
        if k_w is not None:
            kwp, wf2 = self._weight(k_w, "k norm weight", d)
            if q_w is not None and wf2 != wf:
                raise KernelError("qkv_post: q and k norm weights must have the same type")
            wf = wf2
        rot_half = 0
        if cos is not None:
            max_pos, rot_half = cos.shape
            self._elem(cos, "cos", max_pos, rot_half)
            self._elem(sin, "sin", max_pos, rot_half)
            self._i32(positions, "positions", T)
        kcp = vcp = None
        if nkv:
            pages = k_cache.shape[0]
            kcp = self._elem(k_cache, "k cache", pages, nkv, page_size, d)
            vcp = self._elem(v_cache, "v cache", pages, nkv, d, page_size)
            self._i32(slots, "slots", T)
        self._call(self.lib.vk_qkv_post, qkv.data_ptr(), W, q_out.data_ptr() if nq else None, kcp, vcp, qwp, kwp, wf,
                   cos.data_ptr() if cos is not None else None, sin.data_ptr() if sin is not None else None, rot_half,
                   positions.data_ptr() if positions is not None else None,
                   slots.data_ptr() if slots is not None else None, T, nq, nkv, d, page_size, float(eps),
                   self._stream())
        return q_out

    def attn_scratch_floats(self, items: int, nq: int, d: int, nseg: int) -> int:
        """float32 elements of scratch that decode attention (mode 1) needs for ``items`` decoded tokens."""
        return int(self.lib.vk_attn_scratch_floats(items, nq, d, nseg))

    def paged_attention(self, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                        block_table: torch.Tensor, cu_q: torch.Tensor, k_len: torch.Tensor, items: torch.Tensor,
                        *, mode: int, scale: float, window: int = 0, max_k_len: int,
                        nseg: int = 0, scratch: torch.Tensor | None = None,
                        out: torch.Tensor | None = None) -> torch.Tensor:
        """Attention of the rows named by ``items`` over the paged cache (see attention.hip).

        items [n, 2] = (sequence, first row).  mode 0: an item is up to ATTN_ITEM_ROWS consecutive new
        rows of its sequence; modes 2, 6, 8 and 9: the same through a named kernel (same bits); mode 1: an item
        is a single decoded token; modes 3, 4, 5, 7: the same through a named kernel (same bits; see
        attention.hip).  ``max_k_len`` is the host's bound on k_len; the block table must cover it."""
        T, nq, d = q.shape
        pages, nkv, P, d2 = k_cache.shape
        S, W = block_table.shape
        self._elem(q, "q", T, nq, d)
        self._elem(k_cache, "k cache", pages, nkv, P, d)
        self._elem(v_cache, "v cache", pages, nkv, d, P)
        self._i32(block_table, "block table", S, W)
        self._i32(cu_q, "cu_q", S + 1)
        self._i32(k_len, "k_len", S)
        n_items = items.shape[0]
        self._i32(items, "items", n_items, 2)
        if W * P < max_k_len:
            raise KernelError(f"attention: block table of {W} pages of {P} does not cover {max_k_len} keys")
        out = torch.empty_like(q) if out is None else out
        self._elem(out, "out", T, nq, d)
        sp = None
        if mode in (1, 3, 4, 5, 7):
            need_seg = -(-max_k_len // SEGMENT_KEYS)
            if nseg < need_seg:
                raise KernelError(f"attention: {nseg} segments do not cover {max_k_len} keys")
            need = self.attn_scratch_floats(n_items, nq, d, nseg)
            if scratch is None or scratch.numel() < need:
                raise KernelError(f"attention: scratch of {need} floats needed")
            sp = self._f32(scratch, "scratch")
        self._call(self.lib.vk_paged_attention, out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                   block_table.data_ptr(), W, cu_q.data_ptr(), k_len.data_ptr(), items.data_ptr(), n_items, mode,
                   nseg, sp, T, nq, nkv, d, P, window, float(scale), self._stream())
        return out

    def sample(self, logits: torch.Tensor, temps: torch.Tensor | None = None, uniforms: torch.Tensor | None = None,
               out: torch.Tensor | None = None) -> torch.Tensor:
        """Token ids for each row: argmax, or temperature sampling where temps[r] > 0."""
        R, V = logits.shape
        self._elem(logits, "logits", R, V)
        out = torch.empty(R, dtype=torch.int32, device=logits.device) if out is None else out
        self._i32(out, "out", R)
        tp = up = None
        if temps is not None:
            tp, up = self._f32(temps, "temps", R), self._f32(uniforms, "uniforms", R)
        scratch = torch.empty(self.lib.vk_sample_scratch_words(R), dtype=torch.int32, device=logits.device)
        self._call(self.lib.vk_sample, out.data_ptr(), logits.data_ptr(), tp, up, scratch.data_ptr(), R, V, V,
                   self._stream())
        return out


_CACHE: dict[str, Kernels] = {}


def kernels_for(dtype) -> Kernels:
    name = dtype_name(dtype)
    if name not in _CACHE:
        _CACHE[name] = Kernels(name)
    return _CACHE[name]
