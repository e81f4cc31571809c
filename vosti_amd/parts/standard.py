"""The parts that the Qwen3 dense decoder is made of.

Each formula cites the reference file it follows; the kernels' own sources
carry the details.
"""
from __future__ import annotations

from typing import Mapping

import numpy as np
import torch

from ..cache.host import rotary_inverse_frequencies
from ..config.spec import PartSpec
from ..kernels.ops import ATTN_ITEM_ROWS, Kernels, SEGMENT_KEYS
from .base import (Block, Embedding, FeedForward, Head, HostStep, KVPagesSpec, Mixer, Norm, PagedKV, ParamSpec, Part,
                   PositionEncoding, StepContext, build_part, register_part)


@register_part("embedding", "token_embedding")
class TokenEmbedding(Embedding):
    """h[t] = E[ids[t]], a row copy without scale (src/exec/dense_swiglu_model.rs:271-273)."""

    def __init__(self, kernels: Kernels, vocab_size: int, hidden_size: int):
        super().__init__(kernels)
        self.vocab_size, self.hidden_size = vocab_size, hidden_size
        self.weight: torch.Tensor | None = None

    def params(self):
        return {"weight": ParamSpec((self.vocab_size, self.hidden_size))}

    def load(self, tensors):
        self.weight = tensors["weight"]

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        return self.kernels.embedding(self.weight, ids)


@register_part("norm", "rmsnorm")
class RMSNorm(Norm):
    """y = (x * rsqrt(mean(x^2) + eps)) * w in fp32 (kernels/triton_kernels/rmsnorm.py:63-93);
    with a residual the norm sees the unrounded sum (kernels/triton_kernels/rmsnorm_residual.py:73-125)."""

    def __init__(self, kernels: Kernels, size: int, eps: float):
        super().__init__(kernels)
        self.size, self.eps = size, float(eps)
        self.weight: torch.Tensor | None = None

    def params(self):
        return {"weight": ParamSpec((self.size,), init=("uniform", 0.9, 1.1), keep_f32=True)}

    def load(self, tensors):
        self.weight = tensors["weight"]

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.kernels.rmsnorm(x, self.weight, self.eps)

    def forward_add(self, x: torch.Tensor, residual: torch.Tensor) -> torch.Tensor:
        return self.kernels.add_rmsnorm(x, residual, self.weight, self.eps)


_ROTARY_TABLES: dict[tuple, tuple[torch.Tensor, torch.Tensor]] = {}


@register_part("position", "rotary")
class Rotary(PositionEncoding):
    """Half-rotation rotary encoding with precomputed tables
    (python/vosti_kernels/rotary.py:80-90 for the frequencies, :137-160 for the
    tables, kernels/triton_kernels/rope.py:78-123 for the rotation).

    inv_freq[j] = 1 / theta^(2j / rotary_dim) is computed once on the host in
    fp32 by the native library's routine (csrc/host/rules.h), which the native
    engine calls too, so that both have the same bits; the angles, cosines and
    sines of every position are computed on the GPU in fp32 and stored as elements."""

    def __init__(self, kernels: Kernels, head_dim: int, rotary_dim: int, theta: float, max_positions: int):
        super().__init__(kernels)
        if rotary_dim % 2 or not 0 < rotary_dim <= head_dim:
            raise ValueError(f"rotary width {rotary_dim} must be even and at most the head size {head_dim}")
        self.head_dim, self.rotary_dim, self.theta, self.max_positions = head_dim, rotary_dim, float(theta), max_positions
        self._tables: tuple[torch.Tensor, torch.Tensor] | None = None

    def _ensure(self) -> tuple[torch.Tensor, torch.Tensor]:
        if self._tables is None:
            key = (self.kernels.name, self.rotary_dim, self.theta, self.max_positions, torch.cuda.current_device())
            if key not in _ROTARY_TABLES:
                inv_freq = torch.from_numpy(rotary_inverse_frequencies(self.theta, self.rotary_dim)).to("cuda")
                _ROTARY_TABLES[key] = self.kernels.rope_tables(inv_freq, self.max_positions)
            self._tables = _ROTARY_TABLES[key]
        return self._tables

    @property
    def cos(self) -> torch.Tensor:
        return self._ensure()[0]

    @property
    def sin(self) -> torch.Tensor:
        return self._ensure()[1]

    def apply(self, q, k, positions):
        T, nq, d = q.shape
        nk = k.shape[1]
        kw = dict(d=d, k_cache=None, v_cache=None, page_size=0, q_w=None, k_w=None, eps=0.0, cos=self.cos,
                  sin=self.sin, positions=positions, slots=None)
        q2 = self.kernels.qkv_post(q.view(T, nq * d), nq=nq, nkv=0, q_out=None, **kw)
        k2 = self.kernels.qkv_post(k.view(T, nk * d), nq=nk, nkv=0, q_out=None, **kw)
        return q2, k2


@register_part("mixer", "attention")
class Attention(Mixer):
    """Causal grouped-query attention over the paged cache
    (src/exec/dense_swiglu_decoder.rs:171-367): QKV projection without bias,
    per-head RMSNorm of q and k, rotary encoding, store of k and v, attention,
    output projection.  ``window`` > 0 limits a query to that many last keys.

    q_norm, k_norm and position are parts of their own (``PartSpec`` or None);
    when they are this package's RMSNorm and Rotary the three steps between the
    projections run as one launch."""

    def __init__(self, kernels: Kernels, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 scale: float, window: int = 0, q_norm: PartSpec | None = None, k_norm: PartSpec | None = None,
                 position: PartSpec | None = None):
        super().__init__(kernels)
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        if head_dim % 16 or not 16 <= head_dim <= 256:
            raise ValueError(f"head size {head_dim}: the attention kernels take multiples of 16 from 16 to 256")
        self.hidden_size, self.nq, self.nkv, self.d = hidden_size, num_heads, num_kv_heads, head_dim
        self.scale, self.window = float(scale), int(window)
        self.q_norm = build_part("norm", q_norm, kernels) if q_norm else None
        self.k_norm = build_part("norm", k_norm, kernels) if k_norm else None
        self.position = build_part("position", position, kernels) if position else None
        self.w_qkv: torch.Tensor | None = None
        self.w_o: torch.Tensor | None = None
        self._fused = all(p is None or type(p) is RMSNorm for p in (self.q_norm, self.k_norm)) and (
            self.position is None or type(self.position) is Rotary)
        if self._fused and self.q_norm and self.k_norm and self.q_norm.eps != self.k_norm.eps:
            self._fused = False

    def params(self):
        H, nq, nkv, d = self.hidden_size, self.nq, self.nkv, self.d
        return {"q_proj.weight": ParamSpec((nq * d, H)), "k_proj.weight": ParamSpec((nkv * d, H)),
                "v_proj.weight": ParamSpec((nkv * d, H)), "o_proj.weight": ParamSpec((H, nq * d))}

    def children(self):
        c = {}
        if self.q_norm:
            c["q_norm"] = self.q_norm
        if self.k_norm:
            c["k_norm"] = self.k_norm
        if self.position:
            c["position"] = self.position
        return c

    def load(self, tensors):
        # One launch projects q, k and v (kernels/triton_kernels/qkv_matmul.py:108-211);
        # rows of the fused weight are q's, then k's, then v's.
        self.w_qkv = torch.cat([tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]], dim=0).contiguous()
        self.w_o = tensors["o_proj.weight"]

    def cache_spec(self):
        return KVPagesSpec(self.nkv, self.d, self.window)

    # The attention kernels work on items: a single decoded token, or up to ATTN_ITEM_ROWS consecutive rows
    # of a sequence that brings several tokens.  The item lists are the same for every attention layer.
    step_inputs_key = "attention.items"

    @staticmethod
    def _items(step: HostStep) -> dict:
        m = step.memo.get("attention.items")
        if m is None:
            q = np.asarray(step.q_lens, dtype=np.int32)
            single = q == 1
            seqs = np.nonzero(single)[0].astype(np.int32)
            decode = np.stack([seqs, np.zeros_like(seqs)], axis=1) if seqs.size else np.zeros((0, 2), dtype=np.int32)
            prefill = [(s, off) for s in np.nonzero(~single)[0].tolist() for off in range(0, int(q[s]), ATTN_ITEM_ROWS)]
            decode_keys = int(np.asarray(step.k_lens, dtype=np.int32)[single].max()) if seqs.size else 0
            # Recorded launches must cover every length that the tables can hold.
            bound = step.k_len_bound if step.frozen else decode_keys
            m = {"prefill": np.asarray(prefill, dtype=np.int32).reshape(-1, 2), "decode": decode, "decode_bound": bound,
                 "nseg": -(-bound // SEGMENT_KEYS)}
            step.memo["attention.items"] = m
        return m

    @classmethod
    def _items_arrays(cls, step: HostStep) -> dict:
        m = cls._items(step)
        return {"attention.prefill_items": m["prefill"], "attention.decode_items": m["decode"]}

    def step_inputs(self, step: HostStep):
        return self._items_arrays(step)

    def _gemm_floats(self, T: int) -> int:
        """Workspace with which the two projections of T rows take their faster route, where there is one."""
        k, H = self.kernels, self.hidden_size
        return max(k.gemm_workspace_floats(T, (self.nq + 2 * self.nkv) * self.d, H),
                   k.gemm_workspace_floats(T, H, self.nq * self.d))

    def workspace_floats(self, step: HostStep) -> int:
        m = self._items(step)
        need = self._gemm_floats(sum(step.q_lens))
        if m["decode"].shape[0]:
            need = max(need, self.kernels.attn_scratch_floats(m["decode"].shape[0], self.nq, self.d, m["nseg"]))
        return need

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: PagedKV) -> torch.Tensor:
        k = self.kernels
        T = x.shape[0]
        nq, nkv, d = self.nq, self.nkv, self.d
        tables = ctx.groups[cache.group]
        # The projections, the attention of decoded tokens and the next projection use the step's workspace
        # one after the other.
        gemm_floats = self._gemm_floats(T)
        ws = ctx.workspace(gemm_floats) if gemm_floats and ctx.workspace is not None else None
        if cache.writable:
            qkv = k.gemm(x, self.w_qkv, workspace=ws)
        else:
            # The keys and values are an earlier execution's: only q is projected.
            qkv = k.gemm(x, self.w_qkv[: nq * d], workspace=ws)
        if self._fused:
            pos = self.position
            q = k.qkv_post(qkv, nq=nq, nkv=nkv if cache.writable else 0, d=d, q_out=None,
                           k_cache=cache.k, v_cache=cache.v, page_size=cache.page_size,
                           q_w=self.q_norm.weight if self.q_norm else None,
                           k_w=self.k_norm.weight if self.k_norm else None,
                           eps=self.q_norm.eps if self.q_norm else (self.k_norm.eps if self.k_norm else 0.0),
                           cos=pos.cos if pos else None, sin=pos.sin if pos else None,
                           positions=ctx.positions, slots=tables.slots)
        else:
            q = self._unfused(qkv, ctx, cache, tables)
        out = torch.empty_like(q)
        m = self._items(ctx.host)
        prefill_items, decode_items = ctx.inputs["attention.prefill_items"], ctx.inputs["attention.decode_items"]
        if prefill_items.shape[0]:
            k.paged_attention(q, cache.k, cache.v, tables.block_table, ctx.cu_q, ctx.k_len, prefill_items, mode=0,
                              scale=self.scale, window=self.window, max_k_len=ctx.host.k_len_bound, out=out)
        if decode_items.shape[0]:
            nseg = m["nseg"]
            scratch = ctx.workspace(k.attn_scratch_floats(decode_items.shape[0], nq, d, nseg))
            k.paged_attention(q, cache.k, cache.v, tables.block_table, ctx.cu_q, ctx.k_len, decode_items, mode=1,
                              scale=self.scale, window=self.window, max_k_len=m["decode_bound"], nseg=nseg,
                              scratch=scratch, out=out)
        return k.gemm(out.view(T, nq * d), self.w_o, workspace=ws)

    def _unfused(self, qkv, ctx, cache, tables):
        """Norm, position encoding and store as separate steps, for parts that are not RMSNorm / Rotary."""
        k = self.kernels
        T = qkv.shape[0]
        nq, nkv, d = self.nq, self.nkv, self.d
        q = qkv[:, : nq * d].contiguous().view(T, nq, d)
        if not cache.writable:
            if self.q_norm:
                q = self.q_norm.forward(q)
            if self.position:
                q, _ = self.position.apply(q, q[:, :1].contiguous(), ctx.positions)
            return q
        kk = qkv[:, nq * d: (nq + nkv) * d].contiguous().view(T, nkv, d)
        vv = qkv[:, (nq + nkv) * d:].contiguous().view(T, nkv, d)
        if self.q_norm:
            q = self.q_norm.forward(q)
        if self.k_norm:
            kk = self.k_norm.forward(kk)
        if self.position:
            q, kk = self.position.apply(q, kk, ctx.positions)
        kv = torch.cat([kk.reshape(T, nkv * d), vv.reshape(T, nkv * d)], dim=1).contiguous()
        k.qkv_post(kv, nq=0, nkv=nkv, d=d, q_out=None, k_cache=cache.k, v_cache=cache.v, page_size=cache.page_size,
                   q_w=None, k_w=None, eps=0.0, cos=None, sin=None, positions=None, slots=tables.slots)
        return q


@register_part("feed_forward", "swiglu")
class SwiGLU(FeedForward):
    """down(silu(gate(x)) * up(x)) without biases (src/exec/dense_swiglu_decoder.rs:396-438);
    gate and up are one projection whose output is rounded before the
    activation (python/vosti_kernels/model_families/qwen3/loader.py:55-58,
    kernels/triton_kernels/silu_mul.py:64-87)."""

    def __init__(self, kernels: Kernels, hidden_size: int, intermediate_size: int):
        super().__init__(kernels)
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.w_gate_up: torch.Tensor | None = None
        self.w_down: torch.Tensor | None = None

    def params(self):
        H, I = self.hidden_size, self.intermediate_size
        return {"gate_proj.weight": ParamSpec((I, H)), "up_proj.weight": ParamSpec((I, H)),
                "down_proj.weight": ParamSpec((H, I))}

    def load(self, tensors):
        self.w_gate_up = torch.cat([tensors["gate_proj.weight"], tensors["up_proj.weight"]], dim=0).contiguous()
        self.w_down = tensors["down_proj.weight"]

    def _gemm_floats(self, T: int) -> int:
        k = self.kernels
        return max(k.gemm_workspace_floats(T, 2 * self.intermediate_size, self.hidden_size, swiglu=True),
                   k.gemm_workspace_floats(T, self.hidden_size, self.intermediate_size))

    def workspace_floats(self, step: HostStep) -> int:
        return self._gemm_floats(sum(step.q_lens))

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        k = self.kernels
        n = self._gemm_floats(x.shape[0])
        ws = ctx.workspace(n) if n and ctx is not None and ctx.workspace is not None else None
        return k.gemm(k.gemm_swiglu(x, self.w_gate_up, workspace=ws), self.w_down, workspace=ws)


@register_part("block", "prenorm")
class PreNormBlock(Block):
    """x += mixer(norm(x)); x += ffn(norm(x)), carried as (hidden, residual) so
    that each add runs inside the next norm
    (src/exec/dense_swiglu_decoder.rs:556-615 first layer, :740-813 others)."""

    def __init__(self, kernels: Kernels, mixer: Mixer, feed_forward: FeedForward, norms: Mapping[str, Norm]):
        super().__init__(kernels)
        missing = {"input", "post_mixer"} - set(norms)
        if missing:
            raise ValueError(f"a prenorm block needs the norms 'input' and 'post_mixer'; missing: {sorted(missing)}")
        self.mixer, self.feed_forward, self.norms = mixer, feed_forward, dict(norms)

    def children(self):
        c = {"mixer": self.mixer, "feed_forward": self.feed_forward}
        c.update({f"norms.{n}": p for n, p in self.norms.items()})
        return c

    def forward(self, hidden, residual, ctx, cache):
        if residual is None:
            residual = hidden
            normed = self.norms["input"].forward(hidden)
        else:
            normed = self.norms["input"].forward_add(hidden, residual)
        mixed = self.mixer.forward(normed, ctx, cache)
        normed = self.norms["post_mixer"].forward_add(mixed, residual)
        return self.feed_forward.forward(normed, ctx), residual


@register_part("head", "linear_head")
class LinearHead(Head):
    """logits = x W^T without bias (src/exec/dense_swiglu_model.rs:976-984).  A head tied to the embedding
    is this same part: the architecture gives its weight the embedding table's tensor name, and the model
    hands both parts the one tensor (python/vosti_kernels/model_families/qwen3/physical.py:131-134).
    ``tied`` only records that for readers of the specification."""

    def __init__(self, kernels: Kernels, vocab_size: int, hidden_size: int, tied: bool = False):
        super().__init__(kernels)
        self.vocab_size, self.hidden_size, self.tied = vocab_size, hidden_size, bool(tied)
        self.weight: torch.Tensor | None = None

    def params(self):
        return {"weight": ParamSpec((self.vocab_size, self.hidden_size))}

    def load(self, tensors):
        self.weight = tensors["weight"]

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.kernels.gemm(x, self.weight)
