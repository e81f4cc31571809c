#!/usr/bin/env python3
"""Decode and prefill throughput of the Qwen3-8B shape with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--layers L]
    python bench.py --shape 0.6b|1.7b|4b|14b|32b    # the same measurement with the layer sizes of another model of the family
    python bench.py --workload mixed14b     # Qwen3-14B shape: 32 prompts of 128 to 4,096 tokens, prefill in portions beside decoding
    python bench.py --workload prefix32b    # Qwen3-32B shape: 64 requests at context 8,192 that share a 1,024-token prefix
    python bench.py --workload aligned      # the reference's aligned phases: batch 4, cached contexts 0 to 16K, 256 new tokens / 127 decode steps

A step is one decode step of the engine (plan, forward, sample, commit) for a
batch of B requests whose prompts of 2,048 random tokens were prefilled through
the same engine.  One JSON line is printed: ``value`` is decoded tokens per
second; ``prefill`` times one 2,048-token prompt (the median of six; the best is
beside it); ``roofline`` prices the decode step's compulsory HBM reads (every
weight once, the live requests' cache) against 8 TB/s; ``points`` holds decode
throughput at batch 1 and 64 and, unless --no-other-shapes, the figures of the
two larger workloads.  Every figure is measured through the engine that
``config.engine`` names (the native one unless --engine python); the one point
measured through the other engine says so in its name.
"""
from __future__ import annotations

import argparse
import os
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
# The two larger shapes of the same family, for the other workloads.
QWEN3_14B = dict(QWEN3_8B, hidden_size=5120, intermediate_size=17408, num_hidden_layers=40, num_attention_heads=40)
QWEN3_32B = dict(QWEN3_8B, hidden_size=5120, intermediate_size=25600, num_hidden_layers=64, num_attention_heads=64)
# The family's other sizes, for --shape (the three small ones tie the head to the embedding).
QWEN3_SHAPES = {
    "0.6b": dict(QWEN3_8B, hidden_size=1024, intermediate_size=3072, num_hidden_layers=28, num_attention_heads=16, tie_word_embeddings=True),
    "1.7b": dict(QWEN3_8B, hidden_size=2048, intermediate_size=6144, num_hidden_layers=28, num_attention_heads=16, tie_word_embeddings=True),
    "4b": dict(QWEN3_8B, hidden_size=2560, intermediate_size=9728, num_hidden_layers=36, tie_word_embeddings=True),
    "8b": QWEN3_8B, "14b": QWEN3_14B, "32b": QWEN3_32B,
}
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
    ap.add_argument("--batch", type=int, default=None, help="requests (default 8; 64 for prefix32b)")
    ap.add_argument("--layers", type=int, default=None, help="layers of the model that is built (default: all of the shape's)")
    ap.add_argument("--shape", default="8b", choices=sorted(QWEN3_SHAPES), help="which size of the family the decode8b workload takes its "
                    "layer sizes from (default: the 8B shape, the one the record is about)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--graphs", type=int, default=1, choices=[0, 1], help="replay decode steps from captured HIP graphs")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points and the prefill timing")
    ap.add_argument("--no-per-kernel", action="store_true", help="skip the timing of the dominant kernels on their own")
    ap.add_argument("--no-other-shapes", action="store_true", help="skip the 14B and 32B workloads that the default record holds as points")
    ap.add_argument("--prompt-tokens", type=int, default=PROMPT_TOKENS,
                    help="context length of the decode measurement (the prefill figure is always of 2,048 tokens)")
    ap.add_argument("--workload", default="decode8b", choices=["decode8b", "mixed14b", "prefix32b", "aligned"])
    ap.add_argument("--engine", default="native", choices=["native", "python"],
                    help="which engine every figure is measured through: the native one (vosti_amd.engine.NativeEngine) or the "
                         "Python step function over the same kernels, cache manager and scheduler")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    if args.steps + args.warmup > GENERATED_TOKENS:
        print(f"bench.py: steps + warmup must not exceed the {GENERATED_TOKENS} generated tokens of the workload")
        return 2

    import torch
    from vosti_amd.config import Qwen3Config
    import tempfile
    from vosti_amd.engine import Engine, NativeEngine
    from vosti_amd.models import build_model
    from vosti_amd.sampling import SamplingParams
    from vosti_amd.weights import random_weights_on_gpu

    if args.workload == "aligned":
        print(json.dumps(aligned_workload(args)), flush=True)
        return 0
    if args.workload != "decode8b":
        print(json.dumps(other_workload(args)), flush=True)
        return 0
    if args.batch is None:
        args.batch = 8
    shape = QWEN3_SHAPES[args.shape]
    shape_name = f"Qwen3-{args.shape.upper()} shape"
    if args.layers is None:
        args.layers = shape["num_hidden_layers"]
    cfg = Qwen3Config(**dict(shape, num_hidden_layers=args.layers))
    # The Python package's model: for the Python engine, and for timing the kernels on their own with its weights.
    need_model = args.engine == "python" or not args.no_points or not args.no_per_kernel
    model = build_model(cfg, args.dtype) if need_model else None
    if model is not None:
        random_weights_on_gpu(model, seed=0)
    torch.cuda.synchronize()
    elem = 2 if args.dtype == "bfloat16" else 4
    dt_name = "bf16" if args.dtype == "bfloat16" else "fp32"
    rng = random.Random(0)
    page = 64
    prompt_tokens = args.prompt_tokens
    pages_per_request = -(-(max(prompt_tokens, PROMPT_TOKENS) + GENERATED_TOKENS + 1) // page)

    def prompt(n=None):
        return [rng.randrange(cfg.vocab_size) for _ in range(prompt_tokens if n is None else n)]

    native_dir = tempfile.TemporaryDirectory()          # what the native engine is given: config.json; the weights are the same random streams
    with open(os.path.join(native_dir.name, "config.json"), "w") as f:
        json.dump(cfg.to_dict(), f)

    def decode_run(B: int, steps: int, warmup: int, per_kernel_into: dict | None = None, which: str | None = None):
        """Seconds per decode step of B requests at the context length, and the mean context over the timed steps."""
        which = which or args.engine
        print(f"bench.py: {shape_name}: {B} requests through the {which} engine", file=sys.stderr, flush=True)
        kw = dict(num_pages=B * pages_per_request, page_size=page, max_num_seqs=B, max_num_batched_tokens=4096,
                  enable_prefix_cache=False, graphs=bool(args.graphs))
        if which == "native":
            eng = NativeEngine(native_dir.name, dtype=args.dtype, random_weights_seed=0, **kw)
        else:
            eng = Engine(model, **kw)
        sp = SamplingParams(max_tokens=GENERATED_TOKENS, ignore_eos=True)
        for _ in range(B):
            eng.add_request(prompt(), sp)
        while len(eng.step()) < B:                       # prefill, two prompts a step, beside the decoding of those that are through
            pass
        for _ in range(warmup):
            assert len(eng.step()) == B
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            eng.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        ctx = prompt_tokens + warmup + 1 + (steps - 1) / 2.0          # mean keys per request over the timed steps
        if per_kernel_into is not None:
            try:
                from vosti_amd.cache import CachePool
                pool = eng.pool if which == "python" else CachePool(model, page_size=page, num_pages=B * pages_per_request, num_slots=B + 1)
                per_kernel_into["decode"] = kernel_times(model, cfg, pool, B, int(ctx), elem, decode=True)
                del pool
            except Exception as e:      # the step's own figures stand without these
                per_kernel_into["decode"] = {"error": f"{type(e).__name__}: {e}"}
        del eng
        torch.cuda.empty_cache()
        return dt / steps, ctx

    def prefill_run(reps: int = 6):
        """Seconds for one prompt of 2,048 tokens to its first token, through the engine: every run of one engine (the
        first, untimed, loads the kernels), each a new request on pages that the one before gave back."""
        kw = dict(num_pages=pages_per_request, page_size=page, max_num_seqs=1, max_num_batched_tokens=PROMPT_TOKENS,
                  enable_prefix_cache=False)
        if args.engine == "native":
            eng = NativeEngine(native_dir.name, dtype=args.dtype, random_weights_seed=0, **kw)
        else:
            eng = Engine(model, **kw)
        times = []
        for i in range(reps + 1):
            eng.add_request(prompt(PROMPT_TOKENS), SamplingParams(max_tokens=1))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            out = eng.step()
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            assert len(out) == 1 and not eng.has_unfinished()
        del eng
        torch.cuda.empty_cache()
        return sorted(times[1:])

    kernels: dict = {}
    step_s, ctx = decode_run(args.batch, args.steps, args.warmup, None if args.no_per_kernel else kernels)
    value = args.batch / step_s
    bytes_step = decode_bytes(cfg, args.batch, ctx, elem)
    achieved = bytes_step / step_s / 1e9
    record = {
        "metric": f"decode tok/s at batch {args.batch} (+ batch 1/64 and prefill tok/s at 2,048 tok), {shape_name}",
        "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dt_name, "data": "synthetic: seeded random token prompts, seeded random weights",
        "config": {"model": shape_name, "layers": args.layers, "layers_of_model": shape["num_hidden_layers"],
                   "hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size,
                   "q_heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                   "vocab_size": cfg.vocab_size, "global_batch": args.batch, "seq_len": prompt_tokens + GENERATED_TOKENS,
                   "prompt_tokens": prompt_tokens, "context_at_timing": round(ctx), "page_size": page,
                   "parallelism": "single GPU", "graphs": bool(args.graphs), "engine": args.engine},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not args.no_points:
        times = prefill_run()
        t = (times[len(times) // 2 - 1] + times[len(times) // 2]) / 2 if len(times) % 2 == 0 else times[len(times) // 2]
        flops = prefill_flops(cfg, PROMPT_TOKENS)
        record["prefill"] = {"value": round(PROMPT_TOKENS / t, 1), "tokens": PROMPT_TOKENS, "ms": round(t * 1e3, 3),
                             "frac": round(flops / t / PEAK_FLOPS[dt_name], 4), "of": "median of six", "best_ms": round(times[0] * 1e3, 3),
                             "engine": args.engine}
        points = {}
        other_shapes = not args.no_other_shapes and args.shape == "8b" and args.dtype == "bfloat16"

        def other_point(workload):
            """One of the two larger workloads of the same family, whole models, as points of this record (their own
            records: --workload mixed14b, --workload prefix32b)."""
            other_args = argparse.Namespace(**dict(vars(args), workload=workload, layers=None, batch=None, steps=16, warmup=8))
            try:
                r = other_workload(other_args)
            except Exception as e:          # the record's own figures stand without these
                points[workload + "_error"] = f"{type(e).__name__}: {e}"
                return
            if workload == "mixed14b":
                points.update(mixed14b_tokens_per_s=r["value"], mixed14b_output_tokens_per_s=r["output"]["value"],
                              mixed14b_wall_s=r["output"]["wall_s"])
            else:
                points.update(prefix32b_decode_b64_tokens_per_s=r["value"], prefix32b_ms_per_step=r["ms_per_step"],
                              prefix32b_roofline_frac=r["roofline"]["frac"], prefix32b_prefill_tokens_per_s=r["prefill"]["value"])

        # The mixed workload is a few seconds of matrix work, and the card's clock drops for a while after a long
        # stretch of that (the same workload right after the batch 64 prompts and the kernels' own timing: 16 k
        # tokens a second instead of 21 k): it runs here, while little such work lies behind.
        if other_shapes:
            other_point("mixed14b")
        # At batch 1 the first forty or so steps after a new engine's prompt run 4 % slower than the rest (4.35 against
        # 4.18 ms), whichever engine runs them: the point is taken after 48 untimed steps, and the steps right after
        # the prompt and those after 150 steps stand beside it.
        for B, name, warm in ((1, "decode_b1", 48), (1, "decode_b1_first_steps", 2), (1, "decode_b1_after_150_steps", 150), (64, "decode_b64", 48)):
            s, _ = decode_run(B, min(args.steps, 32), max(args.warmup, warm) if warm >= 48 else warm)
            points[name] = round(B / s, 2)
        # The same steps through the other engine: what the Python host code between two steps costs.
        other = "python" if args.engine == "native" else "native"
        s, _ = decode_run(args.batch, args.steps, args.warmup, which=other)
        points[f"decode_b{args.batch}_{other}_engine"] = round(args.batch / s, 2)
        record["points"] = points
        if not args.no_per_kernel:
            try:
                from vosti_amd.cache import CachePool
                pool = CachePool(model, page_size=page, num_pages=PROMPT_TOKENS // page, num_slots=1)
                kernels["prefill"] = kernel_times(model, cfg, pool, PROMPT_TOKENS, PROMPT_TOKENS, elem, decode=False)
            except Exception as e:
                kernels["prefill"] = {"error": f"{type(e).__name__}: {e}"}
    if kernels:
        record["kernels"] = kernels
    if not args.no_points and other_shapes:
        del model
        torch.cuda.empty_cache()
        other_point("prefix32b")            # last: its prompts alone are half a minute of matrix work
    print(json.dumps(record), flush=True)
    return 0


def kernel_times(model, cfg, pool, M: int, keys: int, elem: int, decode: bool) -> dict:
    """The dominant kernels on their own, at the step's shapes: each is recorded once per layer (with that
    layer's weights and cache, so that nothing is warmer than in a step) into a graph, and the graph is
    replayed.  decode: M rows of one token each over ``keys`` keys; else one prompt of M tokens.
    Returns {kernel: {"us": per call, "GBps" or "TFLOPs": achieved, "frac": of the published peak}}."""
    import torch
    k = model.kernels
    L = len(model.layers)
    H, nq, nkv, d, I, V = (cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim,
                           cfg.intermediate_size, cfg.vocab_size)
    dt_name = "bf16" if elem == 2 else "fp32"
    gen = torch.Generator(device="cuda").manual_seed(1)
    rnd = lambda *shape: (torch.randn(*shape, generator=gen, device="cuda") * 0.5).to(k.dtype)
    x, a, m, q = rnd(M, H), rnd(M, nq * d), rnd(M, I), rnd(M, nq, d)
    P = pool.page_size
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")
    if decode:
        W = -(-keys // P)
        table = i32([[s * W + j for j in range(W)] for s in range(M)])
        cu_q, k_len, items = i32(list(range(M + 1))), i32([keys] * M), i32([[s, 0] for s in range(M)])
        nseg = -(-keys // 256)
        scratch = torch.empty(k.attn_scratch_floats(M, nq, d, nseg), dtype=torch.float32, device="cuda")
        attn = lambda c, out: k.paged_attention(q, c.k, c.v, table, cu_q, k_len, items, mode=1, scale=d ** -0.5,
                                                max_k_len=keys, nseg=nseg, scratch=scratch, out=out)
    else:
        W = -(-M // P)
        table = i32([list(range(W))])
        cu_q, k_len = i32([0, M]), i32([M])
        items = i32([[0, o] for o in range(0, M, 128)])
        attn = lambda c, out: k.paged_attention(q, c.k, c.v, table, cu_q, k_len, items, mode=0, scale=d ** -0.5,
                                                max_k_len=M, out=out)
    layers = model.layers
    o_qkv, o_h, o_i, o_attn = k.empty(M, (nq + 2 * nkv) * d), k.empty(M, H), k.empty(M, I), k.empty(M, nq, d)
    # The step's workspace, as the parts ask for it: with it some projections take the route through chunk sums.
    need = max(k.gemm_workspace_floats(M, rows_, K_, swiglu=sw) for rows_, K_, sw in
               (((nq + 2 * nkv) * d, H, False), (H, nq * d, False), (2 * I, H, True), (H, I, False)))
    ws = torch.empty(max(need, 1), dtype=torch.float32, device="cuda")
    head_rows = M if decode else 1
    o_v = k.empty(head_rows, V)
    work = {
        "qkv": (lambda l: k.gemm(x, layers[l].mixer.w_qkv, out=o_qkv, workspace=ws), (nq + 2 * nkv) * d * H, L),
        "attention": (lambda l: attn(pool.entries[l], o_attn), None, L),
        "o": (lambda l: k.gemm(a, layers[l].mixer.w_o, out=o_h, workspace=ws), H * nq * d, L),
        "gate_up": (lambda l: k.gemm_swiglu(x, layers[l].feed_forward.w_gate_up, workspace=ws), 2 * I * H, L),
        "down": (lambda l: k.gemm(m, layers[l].feed_forward.w_down, out=o_h, workspace=ws), H * I, L),
        "lm_head": (lambda l: k.gemm(x[:head_rows], model.head.weight, out=o_v), V * H, 1),
    }
    out = {}
    reps = 5

    def time_calls(fn, calls):
        for l in range(calls):                      # warm: every kernel variant is loaded before the capture
            fn(l)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for l in range(calls):
                fn(l)
        graph.replay()
        torch.cuda.synchronize()
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0.record()
        for _ in range(reps):
            graph.replay()
        t1.record()
        torch.cuda.synchronize()
        return t0.elapsed_time(t1) * 1e3 / (reps * calls)

    # The yardstick for the decode projections: a kernel that only reads the same weights, launch after launch
    # like them (what such reads reach on this machine, well below the 8 TB/s that the fractions are priced at).
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")
    weights = {"qkv": lambda l: layers[l].mixer.w_qkv, "o": lambda l: layers[l].mixer.w_o,
               "gate_up": lambda l: layers[l].feed_forward.w_gate_up, "down": lambda l: layers[l].feed_forward.w_down,
               "lm_head": lambda l: model.head.weight}
    for name, (fn, weight_elems, calls) in work.items():
        us = time_calls(fn, calls)
        rows = head_rows if name == "lm_head" else M
        if name == "attention":
            flops = 4.0 * nq * d * (M * keys if decode else M * (M + 1) / 2)
            nbytes = (M if decode else 1) * keys * 2 * nkv * d * elem
        else:
            flops, nbytes = 2.0 * rows * weight_elems, weight_elems * elem
        if decode or name == "lm_head":      # one row through the head is a read of its weights, whatever the step
            gbps = nbytes / us / 1e3
            out[name] = {"us": round(us, 2), "GBps": round(gbps, 1), "frac": round(gbps / HBM_PEAK_GBS, 3)}
            if name in weights:
                pull_us = time_calls(lambda l, get=weights[name]: k.pull(get(l), sink), calls)
                out[name].update(read_only_us=round(pull_us, 2), frac_of_read_only=round(pull_us / us, 3))
        else:
            tf = flops / us / 1e6
            out[name] = {"us": round(us, 2), "TFLOPs": round(tf, 1), "frac": round(tf * 1e12 / PEAK_FLOPS[dt_name], 3)}
    return out


def progress(text: str, state={"t": 0.0}) -> None:
    """A line on stderr, at most every ten seconds: long runs show that they are alive."""
    now = time.perf_counter()
    if now - state["t"] >= 10.0:
        state["t"] = now
        print(f"bench.py: {text}", file=sys.stderr, flush=True)


def aligned_workload(args) -> dict:
    """The reference's controlled phases (scripts/serving_benchmark/aligned/README.md:9-18, 49-53; docs/artifact.md:232-237),
    through the engine as its own adapter does it (admit all four, then call step): batch 4; cached contexts of 0, 4,096,
    8,192, 12,288 and 16,384 tokens; a prefill wave adds 256 tokens a request and takes one token (throughput = 1,024
    new tokens / the median interval of five waves after two untimed ones, an interval being one engine step between two
    synchronisations); a decode wave times the 127 steps after the first token, every step with the same four requests and
    replayed from a recorded graph.  To have exactly L tokens cached, an untimed donor of L + 1 tokens that differs from the
    measured prompt at token L runs first; the engine's count of reused pages must grow by 4 L / 64 in the timed step."""
    import tempfile
    import torch
    from vosti_amd.config import Qwen3Config
    from vosti_amd.engine import NativeEngine
    from vosti_amd.sampling import SamplingParams

    if args.engine != "native":
        raise SystemExit("bench.py: the aligned phases are measured through the native engine")
    shape = QWEN3_SHAPES[args.shape]
    layers = args.layers if args.layers is not None else shape["num_hidden_layers"]
    cfg = Qwen3Config(**dict(shape, num_hidden_layers=layers))
    elem = 2 if args.dtype == "bfloat16" else 4
    dt_name = "bf16" if args.dtype == "bfloat16" else "fp32"
    page, B, new, out_tokens = 64, 4, 256, 128
    contexts = (0, 4096, 8192, 12288, 16384)
    model_dir = tempfile.TemporaryDirectory()
    with open(os.path.join(model_dir.name, "config.json"), "w") as f:
        json.dump(cfg.to_dict(), f)
    # Four requests of the longest kind and their donors alive at a time; what earlier waves published stays until the room is wanted.
    pages = 3 * B * (-(-(contexts[-1] + new + out_tokens + 2) // page)) + 16
    eng = NativeEngine(model_dir.name, dtype=args.dtype, random_weights_seed=0, num_pages=pages, page_size=page, max_num_seqs=B,
                       max_num_batched_tokens=4096, enable_prefix_cache=True, graphs=bool(args.graphs))
    torch.cuda.synchronize()
    print("bench.py: weights ready", file=sys.stderr, flush=True)
    rng = random.Random(42)
    first = iter(range(1000, cfg.vocab_size))          # distinct first tokens across requests and waves

    def tokens(n):
        return [rng.randrange(cfg.vocab_size) for _ in range(n)]

    def drain():
        while eng.has_unfinished():
            eng.step()

    def cohort(L, own):
        """Four prompts of L cached tokens and `own` new ones; their donors have run and are gone."""
        prefixes = [[next(first)] + tokens(L - 1) if L else [] for _ in range(B)]
        if L:
            for p_ in prefixes:
                eng.add_request(p_ + [0], SamplingParams(max_tokens=1, ignore_eos=True))      # L + 1 tokens: the pages of the first L are published
            drain()
        return [p_ + [next(first)] + tokens(own - 1) for p_ in prefixes]      # token L is not the donor's

    points, detail = {}, {}
    for L in contexts:
        # ---- prefill: 256 new tokens a request, one token out ----
        intervals = []
        for wave in range(2 + 5):
            prompts = cohort(L, new)
            hits = eng.stats()["prefix_hits"]
            for p_ in prompts:
                eng.add_request(p_, SamplingParams(max_tokens=1, ignore_eos=True))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            emitted = eng.step()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            if len(emitted) != B or eng.has_unfinished():
                raise RuntimeError(f"aligned prefill at context {L}: the four requests did not run as one step")
            if eng.stats()["prefix_hits"] - hits != B * (L // page):
                raise RuntimeError(f"aligned prefill at context {L}: {eng.stats()['prefix_hits'] - hits} pages reused, {B * (L // page)} expected")
            if wave >= 2:
                intervals.append(dt)
        intervals.sort()
        med = intervals[len(intervals) // 2]
        points[f"prefill_ctx{L}"] = round(B * new / med, 1)
        detail[f"prefill_ctx{L}_ms"] = [round(x * 1e3, 3) for x in intervals]
        progress(f"aligned: context {L}: prefill {points[f'prefill_ctx{L}']} tok/s")
        # ---- decode: one new token a request, then 127 timed steps ----
        rates = []
        for wave in range(1 + 2):
            prompts = cohort(L, 1)
            for p_ in prompts:
                eng.add_request(p_, SamplingParams(max_tokens=out_tokens, ignore_eos=True))
            if len(eng.step()) != B:                   # the first token of each: outside the timing
                raise RuntimeError(f"aligned decode at context {L}: the first step did not emit for all four")
            before = eng.stats()["graph_stats"]
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(out_tokens - 1):
                if len(eng.step()) != B:
                    raise RuntimeError(f"aligned decode at context {L}: a step did not emit for all four")
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            after = eng.stats()["graph_stats"]
            if eng.has_unfinished():
                raise RuntimeError("aligned decode: requests left after 128 tokens")
            replayed_only = after["eager"] == before["eager"] and after["captured"] == before["captured"]
            if wave >= 1:
                if args.graphs and not replayed_only:
                    raise RuntimeError(f"aligned decode at context {L}: a timed step was recorded or ran eagerly")
                rates.append(B * (out_tokens - 1) / dt)
        rates.sort()
        points[f"decode_ctx{L}"] = round(rates[len(rates) // 2], 1)
        progress(f"aligned: context {L}: decode {points[f'decode_ctx{L}']} tok/s")
    name = f"Qwen3-{args.shape.upper()} shape"
    layers_w, head_w = gemm_params(cfg)
    kv_token = 2 * cfg.num_key_value_heads * cfg.head_dim * cfg.num_hidden_layers
    step_s = B / points["decode_ctx4096"]
    read = (layers_w + head_w + B * (4096 + 1 + out_tokens / 2) * kv_token) * elem
    flops4k = 2.0 * B * new * layers_w + 2.0 * B * head_w + 4.0 * cfg.num_attention_heads * cfg.head_dim * B * new * (4096 + new / 2) * cfg.num_hidden_layers
    t4k = B * new / points["prefill_ctx4096"]
    return {"metric": f"aligned phases at batch 4 (the reference's method): decode tok/s over 127 steps at cached context 4,096, {name}",
            "value": points["decode_ctx4096"], "unit": "tokens/s", "n_gpus": 1, "steps": out_tokens - 1, "warmup": 1,
            "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dt_name,
            "data": "synthetic: seeded random token prompts (seed 42), seeded random weights",
            "config": {"model": name, "layers": layers, "layers_of_model": shape["num_hidden_layers"], "hidden_size": cfg.hidden_size,
                       "intermediate_size": cfg.intermediate_size, "q_heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                       "head_dim": cfg.head_dim, "vocab_size": cfg.vocab_size, "global_batch": B, "new_prefill_tokens": new,
                       "output_tokens": out_tokens, "page_size": page, "parallelism": "single GPU", "graphs": bool(args.graphs),
                       "engine": "native", "prefill_waves": "2 untimed + 5", "decode_waves": "1 untimed + 2"},
            "prefill": {"value": points["prefill_ctx4096"], "tokens": B * new, "ms": round(t4k * 1e3, 3),
                        "frac": round(flops4k / t4k / PEAK_FLOPS[dt_name], 4), "cached_context": 4096},
            "roofline": {"bound": "hbm", "achieved": round(read / step_s / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(read / step_s / 1e9 / HBM_PEAK_GBS, 4)},
            "points": points, "intervals": detail}


def other_workload(args) -> dict:
    """The two larger shapes with the workloads named for them: a record each, same fields."""
    import torch
    from vosti_amd.config import Qwen3Config
    import tempfile
    from vosti_amd.engine import Engine, NativeEngine
    from vosti_amd.models import build_model
    from vosti_amd.sampling import SamplingParams
    from vosti_amd.weights import random_weights_on_gpu

    shape = QWEN3_14B if args.workload == "mixed14b" else QWEN3_32B
    full_layers = shape["num_hidden_layers"]
    layers = args.layers if args.layers is not None else full_layers
    cfg = Qwen3Config(**dict(shape, num_hidden_layers=layers))
    print(f"bench.py: {args.workload}: building {layers} layers for the {args.engine} engine", file=sys.stderr, flush=True)
    native_dir = tempfile.TemporaryDirectory()          # what the native engine is given: config.json; it draws the weights itself
    with open(os.path.join(native_dir.name, "config.json"), "w") as f:
        json.dump(cfg.to_dict(), f)

    def make_engine(**kw):
        if args.engine == "native":
            return NativeEngine(native_dir.name, dtype=args.dtype, random_weights_seed=0, **kw)
        model = build_model(cfg, args.dtype)
        random_weights_on_gpu(model, seed=0)
        return Engine(model, **kw)
    elem = 2 if args.dtype == "bfloat16" else 4
    dt_name = "bf16" if args.dtype == "bfloat16" else "fp32"
    rng = random.Random(1)
    page = 64
    name = "Qwen3-14B shape" if args.workload == "mixed14b" else "Qwen3-32B shape"
    base = {"n_gpus": 1, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dt_name,
            "data": "synthetic: seeded random token prompts, seeded random weights", "unit": "tokens/s"}
    shape_keys = {"model": name, "layers": layers, "layers_of_model": full_layers, "hidden_size": cfg.hidden_size,
                  "intermediate_size": cfg.intermediate_size, "q_heads": cfg.num_attention_heads,
                  "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim, "vocab_size": cfg.vocab_size,
                  "page_size": page, "parallelism": "single GPU", "graphs": bool(args.graphs), "engine": args.engine}

    if args.workload == "mixed14b":
        # 32 prompts of 128 to 4,096 tokens, 128 new tokens each; prompts enter in portions of at most 4,096
        # tokens a step beside the decoding of the requests that are further on.
        n, new = 32, 128
        lengths = [rng.randint(128, 4096) for _ in range(n)]
        prompts = [[rng.randrange(cfg.vocab_size) for _ in range(L)] for L in lengths]
        pages = sum(-(-(L + new + 1) // page) for L in lengths) + 8
        eng = make_engine(num_pages=pages, page_size=page, max_num_seqs=n, max_num_batched_tokens=4096,
                          enable_prefix_cache=False, graphs=bool(args.graphs))
        torch.cuda.synchronize()
        print("bench.py: weights ready", file=sys.stderr, flush=True)
        sp = SamplingParams(max_tokens=new, ignore_eos=True)
        for p_ in prompts:
            eng.add_request(p_, sp)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        steps = emitted = 0
        while eng.has_unfinished():
            emitted += len(eng.step())
            steps += 1
            progress(f"step {steps}, {emitted} tokens out")
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert emitted == n * new
        layers_w, head_w = gemm_params(cfg)
        flops = 2.0 * (sum(lengths) + n * new) * layers_w + 2.0 * n * new * head_w
        record = dict(base, metric="tokens/s through a mixed batch: 32 prompts of 128-4,096 tokens in portions beside decoding, Qwen3-14B shape",
                      value=round((sum(lengths) + emitted) / dt, 1), steps=steps, warmup=0, ms_per_step=round(dt / steps * 1e3, 3),
                      config=dict(shape_keys, global_batch=n, prompt_tokens=sum(lengths), new_tokens=emitted, token_budget=4096),
                      output={"value": round(emitted / dt, 1), "wall_s": round(dt, 3)},
                      roofline={"bound": "mfma", "achieved": round(flops / dt / 1e12, 1), "peak": PEAK_FLOPS[dt_name] / 1e12,
                                "unit": "TFLOP/s (projections only)", "frac": round(flops / dt / PEAK_FLOPS[dt_name], 4)})
        return record

    # prefix32b: 64 requests whose prompts share their first 1,024 tokens and go on with 7,168 of their own;
    # the pages of the shared part are computed once and reused.  Decode steps are timed at context ~8,200.
    n, shared_len, own_len = args.batch or 64, 1024, 7168
    shared = [rng.randrange(cfg.vocab_size) for _ in range(shared_len)]
    prompts = [shared + [rng.randrange(cfg.vocab_size) for _ in range(own_len)] for _ in range(n)]
    # The first requests decode while the later ones are still prefilled, one a step: room for that too.
    total = args.steps + args.warmup + n + 16
    pages = shared_len // page + n * (-(-(own_len + total + 1) // page)) + 8
    eng = make_engine(num_pages=pages, page_size=page, max_num_seqs=n, max_num_batched_tokens=8192,
                      enable_prefix_cache=True, graphs=bool(args.graphs))
    torch.cuda.synchronize()
    print("bench.py: weights ready", file=sys.stderr, flush=True)
    sp = SamplingParams(max_tokens=total, ignore_eos=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    # The first request alone, so that its pages are published before the others look for them.
    eng.add_request(prompts[0], sp)
    emitted_tokens = len(eng.step())
    for p_ in prompts[1:]:
        eng.add_request(p_, sp)
    while True:                                             # until every request has its first token: all of them decode
        out = eng.step()
        emitted_tokens += len(out)
        progress(f"prefill: {len(out)} requests decoding")
        if len(out) == n:
            break
    torch.cuda.synchronize()
    prefill_s = time.perf_counter() - t0
    print(f"bench.py: prefill done in {prefill_s:.1f} s", file=sys.stderr, flush=True)
    for _ in range(args.warmup):
        assert len(eng.step()) == n
    emitted_tokens += args.warmup * n
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        eng.step()
    torch.cuda.synchronize()
    step_s = (time.perf_counter() - t0) / args.steps
    # Mean keys a request reads in a timed step: its prompt, the tokens it had put out before, and the steps so far.
    ctx = shared_len + own_len + emitted_tokens / n + (args.steps - 1) / 2.0
    prefix_hits = eng.stats()["prefix_hits"] if args.engine == "native" else eng.cache.prefix_hits()
    layers_w, head_w = gemm_params(cfg)
    kv_token = 2 * cfg.num_key_value_heads * cfg.head_dim * cfg.num_hidden_layers
    unique = (layers_w + head_w + (n * (ctx - shared_len) + shared_len) * kv_token) * elem     # shared pages once
    record = dict(base, metric=f"decode tok/s at batch {n}, context 8,192, a 1,024-token prefix shared through the page cache, Qwen3-32B shape",
                  value=round(n / step_s, 1), steps=args.steps, warmup=args.warmup, ms_per_step=round(step_s * 1e3, 3),
                  config=dict(shape_keys, global_batch=n, seq_len=shared_len + own_len + total, shared_prefix=shared_len,
                              context_at_timing=round(ctx), reused_prefix_pages=prefix_hits),
                  prefill={"value": round((n * own_len + shared_len) / prefill_s, 1), "tokens": n * own_len + shared_len,
                           "ms": round(prefill_s * 1e3, 1)},
                  roofline={"bound": "hbm", "achieved": round(unique / step_s / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                            "frac": round(unique / step_s / 1e9 / HBM_PEAK_GBS, 4)})
    return record


if __name__ == "__main__":
    sys.exit(main())
