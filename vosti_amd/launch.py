"""Command line of the engine, in the manner of the reference's launcher.

    python -m vosti_amd.launch --kind engine --family qwen3 [-- options]
    python -m vosti_amd.launch --kind random-model --family qwen3 -- --config CONFIG.json --seed N --out DIR

The reference starts its engine example through ``scripts/launch.py --kind engine
--family qwen3`` (scripts/launch.py:17-55) and configures it by environment
variables (examples/support/engine_setup.rs:57-69, 110-118;
examples/support/engine_serving.rs:75-231).  The same variables mean the same
here; each also has a command-line option, which wins:

    MODEL_PATH                 --model-path          model folder (required)
    CUDA_DEVICE                --device              only cuda:0 exists here
    VOSTI_PROMPT_IDS           --prompt-ids          comma-separated token ids (default "9707")
    VOSTI_MAX_TOKENS           --max-tokens          new tokens (default 8)
    VOSTI_IGNORE_EOS           --ignore-eos          presence: do not stop on end tokens
    VOSTI_NUM_BLOCKS           --num-blocks          cache pages (default 32)
    VOSTI_MAX_SEQS             --max-seqs            rows per step (default: the batch size)
    VOSTI_MAX_BATCHED_TOKENS   --max-batched-tokens  tokens per step (default 4096)
    VOSTI_CUDA_GRAPH           --graphs              0/1: replay decode steps from captured HIP graphs
    VOSTI_OUTPUT_TOKENS        --output-tokens       write "index<TAB>ids" lines to this file
    VOSTI_BENCH_INPUT          --bench-input         TSV of MAX_TOKENS<TAB>IDS[<TAB>ARRIVAL_STEP] requests
    VOSTI_BENCH_WARMUP_INPUT   --bench-warmup-input  a TSV of other requests, served first by the same engine
    VOSTI_BENCH_GRAPH_PRIMER_INPUT --bench-graph-primer-input  a third TSV, served before the warm-up, so that the
                                                     recordings of its decode steps exist before anything is timed
    VOSTI_BENCH_CALLS          --bench-calls         JSON of several calls served one after the other by one engine
    VOSTI_BENCH_CALL_RESULTS   --bench-call-results  where their records go (a new JSON file)
    VOSTI_MAX_MODEL_LEN        --max-model-len       longest prompt plus output (default: the model's positions)
    VOSTI_LOGITS_DIGEST                              a file that gets "row sha256" for every sampled logits row
    VOSTI_LOGITS_OBSERVER_DIR                        a folder that gets every sampled logits row as float32 .npy and an index
    VOSTI_ENGINE_STEP_TRACE    --step-trace          append one JSON line per step to this file

Options without a counterpart in the reference: VOSTI_DTYPE / --dtype (bfloat16,
float32), VOSTI_TEMPERATURE / --temperature, VOSTI_SEED / --seed,
VOSTI_PAGE_SIZE / --page-size, VOSTI_PREFIX_CACHE / --prefix-cache (0, 1),
VOSTI_PLUGINS / --plugin (shared libraries that bring part kinds and
architectures to the native engine).

Who serves: the native engine's program (``vosti_amd/_lib/vosti_engine``,
csrc/engine/main.cpp), started as a child process with these options and this
environment, as the reference's launcher starts its engine example.  Only a model
whose architecture or parts exist in Python alone (registered with
``vosti_amd.config.register_architecture`` / ``vosti_amd.parts.register_part``) is
served by the Python step function in this process; the library is asked which
it is.  VOSTI_ENGINE / --engine (auto, native, python) overrides that, for tests.
End tokens come from generation_config.json's ``eos_token_id`` (one to three
ids: python/vosti_kernels/serving_workload.py:78-108); without that file there
are none.  It prints ``MODEL_OUTPUT_TOKEN_IDS=[...]`` like the reference, or a
``BENCH batch=... tok_s=...`` line for prepared requests.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path



def families() -> dict[str, str]:
    """--family names: the ``model_type`` of every registered architecture -> its name (those of the native
    library and its plugins, and those registered in Python)."""
    from .config.registry import model_types
    if os.environ.get("VOSTI_PLUGINS"):
        from .engine.native import load_plugins_from_environment
        load_plugins_from_environment()
    return model_types()


def run_native_program(argv: list[str], family: str, dtype: str) -> int:
    """The native engine's program with the launcher's options and environment, as a child process."""
    import subprocess
    from .kernels import build
    program = build.ensure("engine")
    lib = build.ensure({"bfloat16": "bf16", "float32": "f32"}[dtype])
    args, skip = [], False
    for a in argv:                       # --engine is this launcher's own
        if skip:
            skip = False
        elif a == "--engine":
            skip = True
        elif not a.startswith("--engine="):
            args.append(a)
    return subprocess.run([str(program), "--family", family, *args, "--lib-dir", str(lib.parent)]).returncode


def _env(name: str, default=None):
    v = os.environ.get(name)
    return default if v is None or v == "" else v


def engine_parser() -> argparse.ArgumentParser:
    p = argparse.ArgumentParser(prog="vosti_amd.launch --kind engine", description="Generate tokens for prompts given as token ids.")
    p.add_argument("--model-path", default=_env("MODEL_PATH"))
    p.add_argument("--device", default=_env("CUDA_DEVICE", "cuda:0"))
    p.add_argument("--prompt-ids", default=_env("VOSTI_PROMPT_IDS", "9707"))
    p.add_argument("--max-tokens", type=int, default=int(_env("VOSTI_MAX_TOKENS", 8)))
    p.add_argument("--ignore-eos", action="store_true", default="VOSTI_IGNORE_EOS" in os.environ)
    p.add_argument("--num-blocks", type=int, default=int(_env("VOSTI_NUM_BLOCKS", 32)))
    p.add_argument("--max-seqs", type=int, default=int(_env("VOSTI_MAX_SEQS", 0)))
    p.add_argument("--max-batched-tokens", type=int, default=int(_env("VOSTI_MAX_BATCHED_TOKENS", 4096)))
    p.add_argument("--graphs", type=int, default=int(_env("VOSTI_CUDA_GRAPH", 0)), choices=[0, 1])
    p.add_argument("--output-tokens", default=_env("VOSTI_OUTPUT_TOKENS"))
    p.add_argument("--bench-input", default=_env("VOSTI_BENCH_INPUT"))
    p.add_argument("--bench-warmup-input", default=_env("VOSTI_BENCH_WARMUP_INPUT"))
    p.add_argument("--bench-calls", default=_env("VOSTI_BENCH_CALLS"))
    p.add_argument("--bench-call-results", default=_env("VOSTI_BENCH_CALL_RESULTS"))
    p.add_argument("--max-model-len", type=int, default=int(_env("VOSTI_MAX_MODEL_LEN", 0)))
    p.add_argument("--step-trace", default=_env("VOSTI_ENGINE_STEP_TRACE"))
    p.add_argument("--dtype", default=_env("VOSTI_DTYPE", "bfloat16"), choices=["bfloat16", "float32"])
    p.add_argument("--temperature", type=float, default=float(_env("VOSTI_TEMPERATURE", 0.0)))
    p.add_argument("--seed", type=int, default=int(_env("VOSTI_SEED", 0)))
    p.add_argument("--page-size", type=int, default=int(_env("VOSTI_PAGE_SIZE", 64)))
    p.add_argument("--prefix-cache", type=int, default=int(_env("VOSTI_PREFIX_CACHE", 1)), choices=[0, 1])
    p.add_argument("--bench-graph-primer-input", default=_env("VOSTI_BENCH_GRAPH_PRIMER_INPUT"))
    p.add_argument("--plugin", action="append", default=[], help="a shared library of parts for the native engine (may be repeated)")
    p.add_argument("--engine", default=_env("VOSTI_ENGINE", "auto"), choices=["auto", "native", "python"])
    return p


def parse_ids(text: str) -> list[int]:
    try:
        ids = [int(x) for x in text.replace(" ", "").split(",") if x != ""]
    except ValueError:
        raise SystemExit(f"prompt ids must be comma-separated integers, got {text!r}") from None
    if not ids:
        raise SystemExit("the prompt is empty")
    return ids


def parse_prepared(path: str) -> list[tuple[int, list[int], int]]:
    """MAX_TOKENS<TAB>IDS[<TAB>ARRIVAL_STEP] per line; '#' starts a comment
    (examples/support/engine_benchmark.rs:79-165)."""
    out = []
    for n, line in enumerate(Path(path).read_text().splitlines(), 1):
        if not line.strip() or line.lstrip().startswith("#"):
            continue
        f = line.split("\t")
        if len(f) not in (2, 3):
            raise SystemExit(f"{path}:{n}: expected MAX_TOKENS<TAB>IDS[<TAB>ARRIVAL_STEP]")
        out.append((int(f[0]), parse_ids(f[1]), int(f[2]) if len(f) == 3 else 0))
    if not out:
        raise SystemExit(f"{path} holds no requests")
    return out


def resolve_call_prompts(call: dict, prior: list[tuple[list[list[int]], list[list[int]]]]) -> list[list[int]]:
    """The prompts of one call of a multi-call file: given outright, or built from an earlier call's
    prompt, the first ``count`` tokens that call generated for it, and a suffix
    (examples/support/engine_calls.rs:32-56)."""
    src = call.get("output_prefix_from")
    if src is None:
        return [list(map(int, p)) for p in call.get("prompts", [])]
    if not 0 <= src["call"] < len(prior):
        raise SystemExit("bench calls: 'output_prefix_from' names a call that has not run yet")
    prompts, outputs = prior[src["call"]]
    if not 0 <= src["request"] < len(prompts):
        raise SystemExit("bench calls: 'output_prefix_from' names a request that the call does not have")
    out = outputs[src["request"]]
    if src["count"] > len(out):
        raise SystemExit("bench calls: 'output_prefix_from' wants more tokens than were generated")
    return [prompts[src["request"]] + out[:src["count"]] + [int(t) for t in src.get("suffix", [])]]


def run_calls(engine, path: str, results_path: str | None, eos, args) -> int:
    """Several calls through one engine, one after the other (examples/support/engine_calls.rs:58-123):
    {"prefix_caching": bool, "calls": [{"label", "prompts" | "output_prefix_from", "max_tokens"}]}.
    Without prefix caching the cached pages are dropped before every call.  One record per call goes
    to the results file, and ``CALLS_FINISHED <n>`` is printed."""
    import torch
    from .sampling import SamplingParams
    spec = json.loads(Path(path).read_text())
    calls = spec.get("calls") or []
    if not calls:
        raise SystemExit("bench calls: the file holds no calls")
    if not results_path:
        raise SystemExit("bench calls: VOSTI_BENCH_CALL_RESULTS (or --bench-call-results) is required")
    if Path(results_path).exists():
        raise SystemExit(f"bench calls: {results_path} exists already")
    prior, records, base = [], [], 0
    for index, call in enumerate(calls):
        if engine.has_unfinished():
            raise SystemExit("bench calls: the call before did not finish")
        dropped = 0 if spec.get("prefix_caching") else engine.cache.drop_cached()
        prompts = resolve_call_prompts(call, prior)
        if not prompts or any(not p for p in prompts) or int(call.get("max_tokens", 0)) <= 0:
            raise SystemExit("bench calls: a call has an empty prompt, an empty batch or no output budget")
        os.environ["VOSTI_LOGITS_OBSERVER_PHASE"] = f"call-{index}"
        params = SamplingParams(max_tokens=int(call["max_tokens"]), temperature=args.temperature, seed=args.seed,
                                eos_token_ids=eos, ignore_eos=args.ignore_eos)
        engine._next_id = max(engine._next_id, base)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        outputs = engine.generate(prompts, params)
        wall = time.perf_counter() - t0
        records.append({"label": call.get("label", str(index)), "request_id_base": base, "input_token_ids": prompts,
                        "output_token_ids": outputs, "reclaimed_pages_before_call": dropped,
                        "cache_isolated": not spec.get("prefix_caching"), "cache_page_tokens": engine.pool.page_size,
                        "wall_s": wall, "graph_stats": dict(engine.runner.graph_stats)})
        base += len(prompts)
        prior.append((prompts, outputs))
    with open(results_path, "x") as f:
        json.dump(records, f)
    print(f"CALLS_FINISHED {len(records)}")
    return 0


def eos_ids(model_path: str) -> tuple[int, ...]:
    path = Path(model_path) / "generation_config.json"
    if not path.is_file():
        return ()
    v = json.loads(path.read_text()).get("eos_token_id")
    if v is None:
        return ()
    ids = [v] if isinstance(v, int) else list(v)
    if not 1 <= len(ids) <= 3:
        raise SystemExit("generation_config.json: 'eos_token_id' must hold one to three ids")
    return tuple(int(i) for i in ids)


def run_engine(argv: list[str], family: str) -> int:
    args = engine_parser().parse_args(argv)
    if not args.model_path:
        raise SystemExit("MODEL_PATH (or --model-path) is required")
    if args.device not in ("cuda:0", "cuda"):
        raise SystemExit(f"device {args.device!r}: this engine runs on cuda:0 only")
    which = args.engine
    if which != "python":
        from .engine.native import load_plugin, native_support
        for path in args.plugin:
            load_plugin(path)
        supported, why = native_support(args.model_path)
        if which == "native" and not supported:
            raise SystemExit(f"--engine native: {why}")
        which = "native" if supported else "python"
    if which == "native":
        return run_native_program(argv, family, args.dtype)
    from .config import load_config
    cfg = load_config(args.model_path)
    if cfg.architecture != families()[family]:
        raise SystemExit(f"{args.model_path} holds a {cfg.architecture}, not a {family} model")
    from .engine import Engine
    from .sampling import SamplingParams
    if args.bench_calls:
        requests = []
    elif args.bench_input:
        requests = parse_prepared(args.bench_input)
    else:
        requests = [(args.max_tokens, parse_ids(args.prompt_ids), 0)]
    warmup = parse_prepared(args.bench_warmup_input) if args.bench_input and args.bench_warmup_input else []
    primer = parse_prepared(args.bench_graph_primer_input) if warmup and args.bench_graph_primer_input else []
    eos = eos_ids(args.model_path)
    engine = Engine(args.model_path, dtype=args.dtype, num_pages=args.num_blocks, page_size=args.page_size,
                    max_num_seqs=args.max_seqs or max(len(requests), len(warmup), len(primer), 1 if not args.bench_calls else 8),
                    max_num_batched_tokens=args.max_batched_tokens, enable_prefix_cache=bool(args.prefix_cache),
                    max_model_len=args.max_model_len or None, graphs=bool(args.graphs))
    if args.bench_calls:
        return run_calls(engine, args.bench_calls, args.bench_call_results, eos, args)
    trace = open(args.step_trace, "a") if args.step_trace else None
    import torch

    def cache_counters():
        return engine.cache.prefix_hit_requests(), engine.cache.prefix_hits()

    def serve(reqs, first_seed):
        """(outputs, wall seconds, cache statistics of this workload alone)."""
        params = [SamplingParams(max_tokens=m, temperature=args.temperature, seed=first_seed + i, eos_token_ids=eos,
                                 ignore_eos=args.ignore_eos) for i, (m, _, _) in enumerate(reqs)]
        before = cache_counters()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        outs = engine.generate([ids for _, ids, _ in reqs], params, [a for _, _, a in reqs], trace=trace)
        wall = time.perf_counter() - t0
        after = cache_counters()
        stats = {"admitted_requests": len(reqs), "requests_with_reuse": after[0] - before[0],
                 "reused_prefix_blocks": after[1] - before[1]}
        return outs, wall, stats

    def line(tag, reqs, outs, wall, rate):
        n_out = sum(len(o) for o in outs)
        text = f"{tag} batch={len(reqs)} prompt_tokens={sum(len(i) for _, i, _ in reqs)} output_tokens={n_out} wall_s={wall:.9f}"
        return text + (f" tok_s={n_out / wall:.6f}" if rate else "")

    if primer:
        # An optional third workload, served first in the same engine, so that the captures of the decode steps it
        # walks through exist before the warm-up (examples/support/engine_serving.rs:162-181); nothing is reported of it.
        os.environ["VOSTI_LOGITS_OBSERVER_PHASE"] = "primer"
        serve(primer, args.seed + len(requests) + len(warmup))
    if warmup:
        # The reference serves a disjoint warm-up workload in the same engine before the measured one
        # (examples/support/engine_serving.rs:157-206) and reports both (engine_benchmark.rs:45-76).
        os.environ["VOSTI_LOGITS_OBSERVER_PHASE"] = "warmup"
        w_out, w_wall, w_stats = serve(warmup, args.seed + len(requests))
        print(line("WARMUP", warmup, w_out, w_wall, rate=False))
        print("WARMUP_CACHE_STATS " + json.dumps(w_stats, separators=(",", ":")))
    if warmup:
        os.environ["VOSTI_LOGITS_OBSERVER_PHASE"] = "measured"
    outputs, wall, stats = serve(requests, args.seed)
    if trace:
        trace.close()
    if args.output_tokens:
        Path(args.output_tokens).write_text("".join(f"{i}\t{','.join(map(str, o))}\n" for i, o in enumerate(outputs)))
    if args.bench_input:
        print(line("BENCH", requests, outputs, wall, rate=True))
        stats["preemptions"] = engine.scheduler.preemptions()
        print("CACHE_STATS " + json.dumps(stats, separators=(",", ":")))
    else:
        print(f"MODEL_OUTPUT_TOKEN_IDS={outputs[0]}")
    if args.graphs:
        print("GRAPH_STATS " + json.dumps(engine.runner.graph_stats, separators=(",", ":")))
    return 0


def run_random_model(argv: list[str], family: str) -> int:
    p = argparse.ArgumentParser(prog="vosti_amd.launch --kind random-model",
                                description="Write a model folder (config.json, model.safetensors) with random weights.")
    p.add_argument("--config", required=True, help="a config.json of the architecture")
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--out", required=True)
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    args = p.parse_args(argv)
    import torch
    from .config import config_from_dict
    from .weights import write_random_model
    raw = json.loads(Path(args.config).read_text())
    raw.setdefault("architectures", [families()[family]])
    out = write_random_model(config_from_dict(raw), args.seed, args.out, getattr(torch, args.dtype))
    print(f"wrote {out}")
    return 0


def main(argv: list[str] | None = None) -> int:
    p = argparse.ArgumentParser(description="Launch the engine or write a random-weights model folder.")
    p.add_argument("--kind", required=True, choices=("engine", "random-model"))
    p.add_argument("--family", required=True, choices=sorted(families()))
    p.add_argument("args", nargs=argparse.REMAINDER, help="options of the chosen kind, after --")
    ns = p.parse_args(argv)
    rest = ns.args[1:] if ns.args[:1] == ["--"] else ns.args
    return run_engine(rest, ns.family) if ns.kind == "engine" else run_random_model(rest, ns.family)


if __name__ == "__main__":
    sys.exit(main())
