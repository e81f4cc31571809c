"""A plain, slow implementation of the Qwen3 dense decoder, for tests.

Whole sequences, no cache, no batching, torch on the CPU, one function per
part.  It is written from the reference's formulas (each function cites them)
and shares no code with ``vosti_amd``.  The reference is read, not run.

``dtype`` is the model's storage type.  With ``torch.float32`` nothing is
rounded.  With ``torch.bfloat16`` every tensor the reference stores in the model
type is rounded to it at the same place (``_store``), while the arithmetic
stays in float32 as in the reference's kernels.
"""
from __future__ import annotations

import json
import math
from pathlib import Path

import torch
from safetensors.torch import load_file


def _store(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """What a store in the model type and a reload give, as float32."""
    return x.to(dtype).to(torch.float32)


def embedding(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """o[t, :] = W[ids[t], :], a copy without scale.
    kernels/triton_kernels/embedding.py:57-84; src/exec/dense_swiglu_model.rs:271-273."""
    return table[ids.long()].to(torch.float32)


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float, dtype: torch.dtype) -> torch.Tensor:
    """var = sum(x^2)/N; y = (x * rsqrt(var + eps)) * w, all in float32.
    kernels/triton_kernels/rmsnorm.py:63-93."""
    x = x.to(torch.float32)
    var = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return _store((x * torch.rsqrt(var + eps)) * w.to(torch.float32), dtype)


def add_rms_norm(x: torch.Tensor, residual: torch.Tensor, w: torch.Tensor, eps: float,
                 dtype: torch.dtype) -> tuple[torch.Tensor, torch.Tensor]:
    """h = x + residual in float32; the new residual is h rounded; the norm is
    computed on the unrounded h.  kernels/triton_kernels/rmsnorm_residual.py:73-125."""
    h = x.to(torch.float32) + residual.to(torch.float32)
    var = (h * h).sum(dim=-1, keepdim=True) / h.shape[-1]
    normed = (h * torch.rsqrt(var + eps)) * w.to(torch.float32)
    return _store(normed, dtype), _store(h, dtype)


def linear(x: torch.Tensor, w: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """c = a @ W^T with float32 accumulation, no bias; W in [out, in] layout.
    kernels/triton_kernels/matmul.py:94-147; src/exec/dense_swiglu_decoder.rs:358-367."""
    return _store(x.to(torch.float32) @ w.to(torch.float32).t(), dtype)


def head_rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float, dtype: torch.dtype) -> torch.Tensor:
    """Per token and head: y = x * rsqrt(sum(x^2)/D + eps) * w, w of shape [D]
    shared by all heads.  x: [T, heads, D].  kernels/triton_kernels/qk_norm.py:67-95."""
    x = x.to(torch.float32)
    var = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return _store(x * torch.rsqrt(var + eps) * w.to(torch.float32), dtype)


def rope_tables(max_positions: int, rotary_dim: int, theta: float, dtype: torch.dtype) -> tuple[torch.Tensor, torch.Tensor]:
    """inv_freq = 1 / theta^(arange(0, D, 2)/D) in float32; angle = inv_freq * p;
    cos and sin in float32, then stored in the model type.
    python/vosti_kernels/rotary.py:80-90 and :137-160."""
    inv_freq = 1.0 / (float(theta) ** (torch.arange(0, rotary_dim, 2, dtype=torch.int64).to(torch.float32) / rotary_dim))
    pos = torch.arange(max_positions, dtype=torch.int64).to(torch.float32)
    ang = pos[:, None] * inv_freq[None, :]
    return _store(ang.cos(), dtype), _store(ang.sin(), dtype)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor,
               dtype: torch.dtype) -> torch.Tensor:
    """x1 = x[..., :D/2], x2 = x[..., D/2:]; y1 = x1*cos - x2*sin; y2 = x2*cos + x1*sin,
    with the table row of each token's position.  x: [T, heads, D].
    kernels/triton_kernels/rope.py:78-123."""
    x = x.to(torch.float32)
    half = cos.shape[1]
    c = cos[positions.long()][:, None, :]
    s = sin[positions.long()][:, None, :]
    x1, x2, rest = x[..., :half], x[..., half:2 * half], x[..., 2 * half:]
    return _store(torch.cat([x1 * c - x2 * s, x2 * c + x1 * s, rest], dim=-1), dtype)


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, dtype: torch.dtype,
              window: int = 0, q_positions: torch.Tensor | None = None) -> torch.Tensor:
    """Causal grouped-query attention of one sequence, row by row.

    q: [Tq, nq, D] at positions q_positions (default: the last Tq of the Tk keys,
    i.e. bottom-right aligned); k, v: [Tk, nkv, D] at positions 0..Tk-1.  q head h
    reads kv head h * nkv // nq.  Row at position p sees keys max(0, p-window+1)..p
    (all keys 0..p without a window).  Scores (q.k)*scale, softmax with float32
    statistics; the probabilities are rounded to the model type before they
    multiply V, the normaliser is the sum of the unrounded ones; rows that see
    no key give 0.  kernels/triton_kernels/fattn_paged.py:176-179, 198-262."""
    Tq, nq, D = q.shape
    Tk, nkv, _ = k.shape
    q, k, v = q.to(torch.float32), k.to(torch.float32), v.to(torch.float32)
    if q_positions is None:
        q_positions = torch.arange(Tk - Tq, Tk)
    out = torch.zeros(Tq, nq, D, dtype=torch.float32)
    for h in range(nq):
        g = h * nkv // nq
        for r in range(Tq):
            p = int(q_positions[r])
            lo = max(0, p - window + 1) if window > 0 else 0
            if p < lo or p < 0:
                continue
            keys = k[lo:p + 1, g]
            s = (keys @ q[r, h]) * scale
            m = s.max()
            e = torch.exp(s - m)
            out[r, h] = (_store(e, dtype) @ v[lo:p + 1, g]) / e.sum()
    return _store(out, dtype)


def swiglu(gate_up: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """a = gu[:, :I], b = gu[:, I:]; o = a * sigmoid(a) * b in float32.
    kernels/triton_kernels/silu_mul.py:64-87."""
    gu = gate_up.to(torch.float32)
    inter = gu.shape[1] // 2
    a, b = gu[:, :inter], gu[:, inter:]
    return _store(a * torch.sigmoid(a) * b, dtype)


def argmax_token(row: torch.Tensor) -> int:
    """First index of the maximum; NaN counts as the maximum; an empty row gives 0.
    python/vosti_kernels/kernels.py:1079-1104."""
    if row.numel() == 0:
        return 0
    return int(torch.argmax(row).item())


class PlainQwen3:
    """Weights by their names in the checkpoint, config.json keys as they stand."""

    def __init__(self, model_dir: str | Path, dtype: torch.dtype):
        self.cfg = json.loads((Path(model_dir) / "config.json").read_text())
        raw = load_file(str(Path(model_dir) / "model.safetensors"))
        self.dtype = dtype
        self.w = {n: _store(t.to(torch.float32), dtype) for n, t in raw.items()}
        c = self.cfg
        self.L, self.H = c["num_hidden_layers"], c["hidden_size"]
        self.nq, self.nkv = c["num_attention_heads"], c["num_key_value_heads"]
        self.d = c.get("head_dim") or self.H // self.nq
        self.eps, self.theta = c["rms_norm_eps"], c["rope_theta"]
        self.tied = bool(c.get("tie_word_embeddings", False))
        self.cos, self.sin = rope_tables(c["max_position_embeddings"], self.d, self.theta, dtype)

    def layer(self, i: int, hidden: torch.Tensor, residual: torch.Tensor | None,
              positions: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        """One decoder layer on the pair (hidden, residual).
        src/exec/dense_swiglu_decoder.rs:556-615 (first layer: the residual is the
        embedding itself), :740-813 (others), :43-441 (the core)."""
        w, dt = self.w, self.dtype
        p = f"model.layers.{i}."
        if residual is None:
            residual = hidden
            normed = rms_norm(hidden, w[p + "input_layernorm.weight"], self.eps, dt)
        else:
            normed, residual = add_rms_norm(hidden, residual, w[p + "input_layernorm.weight"], self.eps, dt)
        T = normed.shape[0]
        q = linear(normed, w[p + "self_attn.q_proj.weight"], dt).view(T, self.nq, self.d)
        k = linear(normed, w[p + "self_attn.k_proj.weight"], dt).view(T, self.nkv, self.d)
        v = linear(normed, w[p + "self_attn.v_proj.weight"], dt).view(T, self.nkv, self.d)
        q = head_rms_norm(q, w[p + "self_attn.q_norm.weight"], self.eps, dt)
        k = head_rms_norm(k, w[p + "self_attn.k_norm.weight"], self.eps, dt)
        q = apply_rope(q, self.cos, self.sin, positions, dt)
        k = apply_rope(k, self.cos, self.sin, positions, dt)
        attn = attention(q, k, v, self.d ** -0.5, dt)
        proj = linear(attn.reshape(T, self.nq * self.d), w[p + "self_attn.o_proj.weight"], dt)
        normed2, residual = add_rms_norm(proj, residual, w[p + "post_attention_layernorm.weight"], self.eps, dt)
        gate_up = torch.cat([linear(normed2, w[p + "mlp.gate_proj.weight"], dt),
                             linear(normed2, w[p + "mlp.up_proj.weight"], dt)], dim=1)
        down = linear(swiglu(gate_up, dt), w[p + "mlp.down_proj.weight"], dt)
        return down, residual

    def logits(self, ids: list[int], first_position: int = 0) -> torch.Tensor:
        """Logits at every position of one whole sequence: [len(ids), vocab], float32.
        src/exec/dense_swiglu_model.rs:131-1041; a model without layers is
        lm_head(rms_norm(embed)) (:276-359).  ``first_position``: the sequence stands at
        positions first_position, first_position + 1, ... (for the invariance tests)."""
        w, dt = self.w, self.dtype
        t = torch.tensor(ids, dtype=torch.int64)
        positions = torch.arange(first_position, first_position + len(ids))
        hidden, residual = embedding(t, w["model.embed_tokens.weight"]), None
        for i in range(self.L):
            hidden, residual = self.layer(i, hidden, residual, positions)
        if residual is None:
            final = rms_norm(hidden, w["model.norm.weight"], self.eps, dt)
        else:
            final, _ = add_rms_norm(hidden, residual, w["model.norm.weight"], self.eps, dt)
        head = w["model.embed_tokens.weight"] if self.tied else w["lm_head.weight"]
        return linear(final, head, dt)

    def generate_greedy(self, prompt: list[int], n_new: int) -> list[int]:
        ids = list(prompt)
        for _ in range(n_new):
            ids.append(argmax_token(self.logits(ids)[-1]))
        return ids[len(prompt):]
