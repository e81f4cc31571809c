"""Trace replay: the command-line face of the step function (see bin/trace_run)."""
from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path


def build_parser() -> argparse.ArgumentParser:
    p = argparse.ArgumentParser(prog="trace_run", description="Replay token traces through the step function and write logits.")
    p.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    p.add_argument("--dtype", required=True, choices=["bfloat16", "float32"],
                   help="bfloat16: the kernels and precisions of serving; float32: everything in true 32-bit")
    p.add_argument("--out", required=True, help="folder for <step>.f32 files")
    p.add_argument("--max-tokens", type=int, required=True,
                   help="most tokens live requests hold at any time, each request rounded up to a page")
    p.add_argument("--page-size", type=int, default=64, help="tokens per cache page (a power of two, default 64)")
    p.add_argument("--max-requests", type=int, default=8, help="most requests alive at a time (state slots)")
    p.add_argument("--prefix-cache", action="store_true",
                   help="a request whose first tokens equal full pages that an earlier request left reuses those pages: "
                        "feed such a request its tokens from the first uncached one on (--prefix-report tells which)")
    p.add_argument("--engine", default="auto", choices=["auto", "native", "python"],
                   help="which step function runs the trace: the native engine's (csrc/engine/runner.cpp), or the Python one "
                        "(engine/step.py) for a model whose parts exist in Python alone; auto asks the library which it is. "
                        "The same kernels, cache manager and logits")
    p.add_argument("--plugin", action="append", default=[], help="a shared library of parts for the native engine (may be repeated)")
    p.add_argument("--prefix-report", default=None,
                   help="a file that gets one line '<id> <cached tokens>' when a request with a 'prompt' field is first seen")
    return p


def main(argv: list[str] | None = None) -> int:
    args = build_parser().parse_args(argv)
    print("trace_run: loading (native code is compiled at first use)", file=sys.stderr, flush=True)
    import numpy as np
    import torch

    if not torch.cuda.is_available():
        print("trace_run: no GPU visible; this engine has no CPU path", file=sys.stderr)
        return 2
    page = args.page_size
    num_pages = max(1, -(-args.max_tokens // page))
    which = args.engine
    if which != "python":
        from .native import load_plugin, load_plugins_from_environment, native_support
        load_plugins_from_environment()
        for path in args.plugin:
            load_plugin(path)
        supported, why = native_support(args.model)
        if which == "native" and not supported:
            print(f"trace_run: --engine native: {why}", file=sys.stderr)
            return 2
        which = "native" if supported else "python"
    if which == "native":
        from .native import NativeEngine
        native = NativeEngine(args.model, dtype=args.dtype, num_pages=num_pages, page_size=page, max_num_seqs=args.max_requests,
                              enable_prefix_cache=args.prefix_cache, graphs=False)
        add_request, has_request, finish = native.trace_add_request, native.trace_has_request, native.trace_finish

        def step_logits(entries):
            return native.trace_step(entries)
    else:
        from ..cache import CachePool
        from ..models import load_model
        from .step import ModelRunner, StepEntry

        model = load_model(args.model, args.dtype)
        pool = CachePool(model, page_size=page, num_pages=num_pages, num_slots=args.max_requests,
                         prefix_cache=args.prefix_cache)
        runner = ModelRunner(model, pool)
        add_request, has_request, finish = runner.cache.add_request, runner.cache.has_request, runner.finish

        def step_logits(entries):
            logits = runner.step([StepEntry(*e) for e in entries])
            if logits.shape[0] == 0:
                torch.cuda.synchronize()
                return np.empty((0, 0), dtype=np.float32)
            return model.kernels.to_f32(logits).cpu().numpy()
    report = open(args.prefix_report, "a") if args.prefix_report else None
    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)
    ids: dict[str, int] = {}     # request names -> numbers; a name may come back after it ended
    fed: dict[str, int] = {}     # request names -> tokens the request holds so far (cached prefix included)
    next_id = 0
    print("trace_run: ready", file=sys.stderr, flush=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = []
        for e in rec.get("entries", []):
            name = str(e["id"])
            if not e.get("tokens"):
                # Nothing to run for this request in this step: the same as leaving it out.
                if e.get("want"):
                    raise SystemExit(f"trace_run: step {step}: request {name} asks for logits but brings no tokens")
                continue
            if name not in ids:
                ids[name] = next_id
                next_id += 1
                if args.prefix_cache and "prompt" in e:
                    # The whole prompt is announced so that cached pages can be matched; the entry's tokens
                    # must then start right after the cached ones, which are not computed again.
                    cached = add_request(ids[name], [int(t) for t in e["prompt"]])
                    if report:
                        report.write(f"{name} {cached}\n")
                        report.flush()
                    skip = cached - int(e.get("start", 0))
                    if skip < 0:
                        raise SystemExit(f"trace_run: request {name} starts at {e.get('start', 0)} but {cached} tokens are cached")
                    e = dict(e, tokens=e["tokens"][skip:], want=[w - skip for w in e.get("want", []) if w >= skip])
                    fed[name] = cached
                else:
                    fed[name] = int(e.get("start", 0)) if "start" in e else 0
            entries.append((ids[name], [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])]))
        # Which row of the step's file is which: [request id, position of the token in the request] per wanted place.
        index = []
        for e, (rid, tokens, want) in zip([e for e in rec.get("entries", []) if e.get("tokens")], entries):
            name = str(e["id"])
            index += [[e["id"], fed.get(name, 0) + w] for w in want]
            fed[name] = fed.get(name, 0) + len(tokens)
        logits = step_logits(entries)
        if logits.shape[0] > 0:
            logits.astype("<f4", copy=False).tofile(str(out_dir / f"{step}.f32"))
            (out_dir / f"{step}.json").write_text(json.dumps({"step": step, "rows": index, "vocab": int(logits.shape[1])}))
        for name in rec.get("end", []):
            name = str(name)
            fed.pop(name, None)
            if name in ids:
                rid = ids.pop(name)
                if has_request(rid):
                    finish(rid)
        print(f"done {step}", flush=True)
    return 0
