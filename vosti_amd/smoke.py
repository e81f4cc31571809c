"""A few tokens from a tiny random model on cuda:0, checked against a plain forward pass."""
from __future__ import annotations

import tempfile

import torch


def _plain_next_token(w: dict, cfg, ids: list[int]) -> int:
    """Greedy next token by a plain float32 forward pass of the whole sequence (torch, no cache)."""
    H, nq, nkv, d, eps = cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.rms_norm_eps

    def norm(x, g):
        return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * g
    T = len(ids)
    inv = 1.0 / (cfg.rope_theta ** (torch.arange(0, d, 2, dtype=torch.int64).float() / d))
    ang = torch.arange(T).float()[:, None] * inv[None]
    cos, sin = ang.cos()[:, None], ang.sin()[:, None]

    def rope(x):
        a, b = x[..., : d // 2], x[..., d // 2:]
        return torch.cat([a * cos - b * sin, b * cos + a * sin], -1)
    x = w["model.embed_tokens.weight"][torch.tensor(ids)]
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        n = norm(x, w[p + "input_layernorm.weight"])
        q = rope(norm((n @ w[p + "self_attn.q_proj.weight"].t()).view(T, nq, d), w[p + "self_attn.q_norm.weight"]))
        k = rope(norm((n @ w[p + "self_attn.k_proj.weight"].t()).view(T, nkv, d), w[p + "self_attn.k_norm.weight"]))
        v = (n @ w[p + "self_attn.v_proj.weight"].t()).view(T, nkv, d)
        k, v = k.repeat_interleave(nq // nkv, 1), v.repeat_interleave(nq // nkv, 1)
        s = torch.einsum("qhd,khd->hqk", q, k) * d ** -0.5
        s = s.masked_fill(~torch.ones(T, T).tril().bool(), float("-inf"))
        a = torch.einsum("hqk,khd->qhd", torch.softmax(s, -1), v).reshape(T, nq * d)
        x = x + a @ w[p + "self_attn.o_proj.weight"].t()
        n = norm(x, w[p + "post_attention_layernorm.weight"])
        g, u = n @ w[p + "mlp.gate_proj.weight"].t(), n @ w[p + "mlp.up_proj.weight"].t()
        x = x + (torch.nn.functional.silu(g) * u) @ w[p + "mlp.down_proj.weight"].t()
    head = w["model.embed_tokens.weight"] if cfg.tie_word_embeddings else w["lm_head.weight"]
    return int(torch.argmax(norm(x[-1], w["model.norm.weight"]) @ head.t()))


def run_smoke() -> None:
    from safetensors.torch import load_file

    from .config import Qwen3Config
    from .engine import Engine
    from .sampling import SamplingParams
    from .weights import write_random_model

    if not torch.cuda.is_available():
        raise RuntimeError("smoke() needs the GPU: this engine has no CPU path")
    cfg = Qwen3Config(vocab_size=503, hidden_size=96, intermediate_size=224, num_hidden_layers=3, num_attention_heads=8,
                      num_key_value_heads=2, head_dim=32, max_position_embeddings=256, rms_norm_eps=1e-5, rope_theta=1e6,
                      tie_word_embeddings=False)
    with tempfile.TemporaryDirectory() as d:
        write_random_model(cfg, 1, d)
        w = {n: t.float() for n, t in load_file(f"{d}/model.safetensors").items()}
        prompts = [[5, 17, 3, 99, 250], list(range(100, 170))]
        for dtype in ("float32", "bfloat16"):
            engine = Engine(d, dtype=dtype, num_pages=16, page_size=16, max_num_seqs=2)
            outs = engine.generate(prompts, SamplingParams(max_tokens=6))
            print(f"smoke {dtype}: {outs}", flush=True)
            if dtype == "float32":
                for prompt, out in zip(prompts, outs):
                    ids = list(prompt)
                    for tok in out:
                        want = _plain_next_token(w, cfg, ids)
                        if tok != want:
                            raise AssertionError(f"smoke: engine emitted {tok}, the plain forward pass {want}, after {len(ids)} tokens")
                        ids.append(tok)
            loaded = [engine.kernels.path]
            print(f"smoke {dtype}: native library {loaded[0]}", flush=True)
    print("smoke ok", flush=True)
