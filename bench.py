#!/usr/bin/env python3
"""Decode and prefill throughput of the Qwen3-8B shape with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--layers L]

A step is one decode step of the engine (plan, forward, sample, commit) for a
batch of B requests whose prompts of 2,048 random tokens were prefilled through
the same engine.  One JSON line is printed: ``value`` is decoded tokens per
second; ``prefill`` times one 2,048-token prompt; ``roofline`` prices the decode
step's compulsory HBM reads (every weight once, the live requests' cache)
against 8 TB/s; ``points`` holds decode throughput at batch 1 and 64.
"""
from __future__ import annotations

import argparse
import json
import random
import sys
import time
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parent))

# The shape of Qwen3-8B, the model that the reference quotes its figures on.
QWEN3_8B = dict(vocab_size=151936, hidden_size=4096, intermediate_size=12288, num_hidden_layers=36,
                num_attention_heads=32, num_key_value_heads=8, head_dim=128, max_position_embeddings=40960,
                rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=False)
PROMPT_TOKENS = 2048
GENERATED_TOKENS = 256
HBM_PEAK_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}


def gemm_params(cfg) -> int:
    """Matrix elements a token passes through, per layer and for the head."""
    H, nq, nkv, d, I = cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.intermediate_size
    per_layer = (nq + 2 * nkv) * d * H + H * nq * d + 3 * I * H
    return per_layer * cfg.num_hidden_layers, cfg.vocab_size * H


def prefill_flops(cfg, T: int) -> float:
    layers, head = gemm_params(cfg)
    attn = 4.0 * cfg.num_attention_heads * cfg.head_dim * (T * (T + 1) / 2) * cfg.num_hidden_layers
    return 2.0 * T * layers + 2.0 * head + attn      # logits for the last row only


def decode_bytes(cfg, B: int, ctx: float, elem: int) -> float:
    layers, head = gemm_params(cfg)
    kv = B * ctx * 2 * cfg.num_key_value_heads * cfg.head_dim * cfg.num_hidden_layers
    return (layers + head + kv) * elem


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=QWEN3_8B["num_hidden_layers"])
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--graphs", type=int, default=1, choices=[0, 1], help="replay decode steps from captured HIP graphs")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points and the prefill timing")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    if args.steps + args.warmup > GENERATED_TOKENS:
        print(f"bench.py: steps + warmup must not exceed the {GENERATED_TOKENS} generated tokens of the workload")
        return 2

    import torch
    from vosti_amd.config import Qwen3Config
    from vosti_amd.engine import Engine
    from vosti_amd.models import build_model
    from vosti_amd.sampling import SamplingParams
    from vosti_amd.weights import random_weights_on_gpu

    cfg = Qwen3Config(**dict(QWEN3_8B, num_hidden_layers=args.layers))
    model = build_model(cfg, args.dtype)
    random_weights_on_gpu(model, seed=0)
    torch.cuda.synchronize()
    elem = 2 if args.dtype == "bfloat16" else 4
    dt_name = "bf16" if args.dtype == "bfloat16" else "fp32"
    rng = random.Random(0)
    page = 64
    pages_per_request = -(-(PROMPT_TOKENS + GENERATED_TOKENS + 1) // page)

    def prompt():
        return [rng.randrange(cfg.vocab_size) for _ in range(PROMPT_TOKENS)]

    def decode_run(B: int, steps: int, warmup: int):
        eng = Engine(model, num_pages=B * pages_per_request, page_size=page, max_num_seqs=B, max_num_batched_tokens=4096,
                     enable_prefix_cache=False, graphs=bool(args.graphs))
        sp = SamplingParams(max_tokens=GENERATED_TOKENS, ignore_eos=True)
        for _ in range(B):
            eng.add_request(prompt(), sp)
        while eng.scheduler.num_waiting() or any(eng.cache.length(r) < PROMPT_TOKENS for r in range(eng._next_id - B, eng._next_id)):
            eng.step()                                   # prefill, two prompts a step
        for _ in range(warmup):
            assert len(eng.step()) == B
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            eng.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        ctx = PROMPT_TOKENS + warmup + 1 + (steps - 1) / 2.0          # mean keys per request over the timed steps
        del eng
        torch.cuda.empty_cache()
        return dt / steps, ctx

    def prefill_run(reps: int = 3):
        times = []
        for i in range(reps + 1):
            eng = Engine(model, num_pages=pages_per_request, page_size=page, max_num_seqs=1, max_num_batched_tokens=PROMPT_TOKENS,
                         enable_prefix_cache=False)
            eng.add_request(prompt(), SamplingParams(max_tokens=1))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            out = eng.step()
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            assert len(out) == 1
            del eng
        return min(times[1:])

    step_s, ctx = decode_run(args.batch, args.steps, args.warmup)
    value = args.batch / step_s
    bytes_step = decode_bytes(cfg, args.batch, ctx, elem)
    achieved = bytes_step / step_s / 1e9
    record = {
        "metric": "decode tok/s at batch 8 (+ batch 1/64 and prefill tok/s at 2,048 tok), Qwen3-8B shape",
        "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dt_name, "data": "synthetic: seeded random token prompts, seeded random weights",
        "config": {"model": "Qwen3-8B shape", "layers": args.layers, "layers_of_model": QWEN3_8B["num_hidden_layers"],
                   "hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size,
                   "q_heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                   "vocab_size": cfg.vocab_size, "global_batch": args.batch, "seq_len": PROMPT_TOKENS + GENERATED_TOKENS,
                   "prompt_tokens": PROMPT_TOKENS, "context_at_timing": round(ctx), "page_size": page,
                   "parallelism": "single GPU", "graphs": bool(args.graphs)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not args.no_points:
        t = prefill_run()
        flops = prefill_flops(cfg, PROMPT_TOKENS)
        record["prefill"] = {"value": round(PROMPT_TOKENS / t, 1), "tokens": PROMPT_TOKENS, "ms": round(t * 1e3, 3),
                             "frac": round(flops / t / PEAK_FLOPS[dt_name], 4)}
        points = {}
        for B, name in ((1, "decode_b1"), (64, "decode_b64")):
            s, _ = decode_run(B, min(args.steps, 32), min(args.warmup, 4))
            points[name] = round(B / s, 2)
        record["points"] = points
    print(json.dumps(record), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
