"""The engine end to end: scheduler, step function, sampler, entry points."""
import json
import os
import random
import subprocess
import sys

import pytest
import torch

from conftest import ROOT, TINY
from plain_qwen3 import PlainQwen3

pytestmark = pytest.mark.gpu
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def prompts(name, lengths, seed=3):
    rng = random.Random(seed)
    vocab = TINY[name][0]["vocab_size"]
    return [[rng.randrange(vocab) for _ in range(n)] for n in lengths]


def engine(model_dir, dtype, **kw):
    from vosti_amd.engine import Engine
    return Engine(model_dir, dtype=dtype, **kw)


def check_greedy_against_plain(plain, prompt, out, dtype_name, exact=None):
    """Every emitted token is the plain implementation's argmax of the same history; in bfloat16 a
    token also passes whose plain logit lies below the maximum by no more than twice what the type
    itself costs that row (the plain bfloat16 row against the plain float32 row ``exact`` gives): a
    near tie that a sum in another order can turn."""
    ids = list(prompt)
    for tok in out:
        row = plain.logits(ids)[-1]
        if dtype_name == "float32":
            assert tok == int(torch.argmax(row)), (len(ids), tok)
        else:
            cost = (row - exact.logits(ids)[-1]).abs().max().item()
            assert row[tok] >= row.max() - 2 * cost, (len(ids), tok, cost)
        ids.append(tok)


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_tiny_a_workload_greedy(tiny_dirs, dtype_name):
    """Four requests with prompts of 1, 7, 33 and 64 tokens, greedy, 16 new tokens each."""
    from vosti_amd.sampling import SamplingParams
    ps = prompts("A", [1, 7, 33, 64])
    plain, exact = PlainQwen3(tiny_dirs["A"], DTYPES[dtype_name]), PlainQwen3(tiny_dirs["A"], torch.float32)
    outs = engine(tiny_dirs["A"], dtype_name, num_pages=24, page_size=16, max_num_seqs=4).generate(ps, SamplingParams(max_tokens=16))
    assert [len(o) for o in outs] == [16] * 4
    for p, o in zip(ps, outs):
        check_greedy_against_plain(plain, p, o, dtype_name, exact)
    # Alone, with another page size, a small budget and no prefix cache: the same tokens, bit for bit.
    for i, p in enumerate(ps):
        alone = engine(tiny_dirs["A"], dtype_name, num_pages=8, page_size=32, max_num_seqs=1, max_num_batched_tokens=16,
                       enable_prefix_cache=False).generate([p], SamplingParams(max_tokens=16))
        assert alone[0] == outs[i]


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_tiny_b_workload_temperature_staggered(tiny_dirs, dtype_name):
    """Six requests, prompts of 2 to 120 tokens, temperature 0.8 with a seed per request, 24 new tokens,
    staggered arrival; few pages, so that some requests wait and pages are used again."""
    from vosti_amd.sampling import SamplingParams, uniform_for
    ps = prompts("B", [2, 120, 31, 64, 9, 77])
    params = [SamplingParams(max_tokens=24, temperature=0.8, seed=100 + i) for i in range(6)]
    e = engine(tiny_dirs["B"], dtype_name, num_pages=40, page_size=8, max_num_seqs=3, max_num_batched_tokens=48)
    outs = e.generate(ps, params, arrival_steps=[0, 0, 2, 4, 8, 12])
    assert [len(o) for o in outs] == [24] * 6 and e.cache.num_requests() == 0 and e.cache.check() == ""
    # Each request alone draws the same tokens: nothing depends on the companions or the schedule.
    for i in (0, 1, 4):
        alone = engine(tiny_dirs["B"], dtype_name, num_pages=32, page_size=8, max_num_seqs=1).generate([ps[i]], params[i])
        assert alone[0] == outs[i], i
    # Against the plain implementation: the drawn token's interval of the plain CDF holds the same uniform number.
    # In bfloat16 the interval may be off by what the type itself moves the CDF (plain bfloat16 against
    # plain float32 at that step), twice over: once for each of its ends.
    plain, exact = PlainQwen3(tiny_dirs["B"], DTYPES[dtype_name]), PlainQwen3(tiny_dirs["B"], torch.float32)
    cdf_of = lambda model, ids: torch.cumsum(torch.softmax(model.logits(ids)[-1].double() / 0.8, 0), 0)
    for i in (0, 2):
        ids = list(ps[i])
        for j, tok in enumerate(outs[i]):
            cdf = cdf_of(plain, ids)
            slack = 1e-4 if dtype_name == "float32" else 2 * (cdf - cdf_of(exact, ids)).abs().max().item()
            u = uniform_for(params[i].seed, j)
            lo = cdf[tok - 1].item() if tok else 0.0
            assert lo - slack <= u <= cdf[tok].item() + slack, (i, j, slack)
            ids.append(tok)
    # Different seeds give different continuations; temperature 0 in the same batch stays greedy.
    assert outs[0] != engine(tiny_dirs["B"], dtype_name, num_pages=32, page_size=8).generate([ps[0]], SamplingParams(max_tokens=24, temperature=0.8, seed=7))[0]


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_prefix_cache_hit_equals_cold_run(tiny_dirs, dtype_name):
    from vosti_amd.sampling import SamplingParams
    shared = prompts("B", [70], seed=9)[0]
    a, b = shared + [1, 2, 3], shared + [4]
    sp = SamplingParams(max_tokens=8)
    cold = engine(tiny_dirs["B"], dtype_name, num_pages=32, page_size=8, enable_prefix_cache=False)
    want_b = cold.generate([b], sp)[0]
    warm = engine(tiny_dirs["B"], dtype_name, num_pages=32, page_size=8, enable_prefix_cache=True)
    warm.generate([a], sp)
    assert warm.generate([b], sp)[0] == want_b and warm.cache.prefix_hits() == 8      # 64 of 70 shared tokens


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_long_decoding_equals_whole_prompt(tiny_dirs, dtype_name):
    """200 decoded tokens from a short prompt; then the whole sequence in one step: the logits at every
    decoded position are the same bits, so every emitted token is the whole-prompt argmax."""
    from vosti_amd.engine import StepEntry
    from vosti_amd.sampling import SamplingParams
    p = prompts("B", [5], seed=4)[0]
    e = engine(tiny_dirs["B"], dtype_name, num_pages=40, page_size=8, max_num_seqs=2)
    out = e.generate([p], SamplingParams(max_tokens=200))[0]
    seq = p + out
    logits = e.runner.step([StepEntry(12345, seq[:-1], list(range(len(p) - 1, len(seq) - 1)))])
    e.runner.finish(12345)
    assert e.kernels.sample(logits).cpu().tolist() == out


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_schedule_stress(tiny_dirs, dtype_name):
    """Prompts of 17 to 385 tokens around page and tile edges, 16 new tokens each, four rows and 128
    tokens a step, staggered arrival (the reference's schedule stress,
    scripts/determinism_tests/schedule_stress.py:20-106): with many pages or few, with or without graph
    replay, every request gets the tokens of a run on its own."""
    from vosti_amd.sampling import SamplingParams
    ps = prompts("C", [17, 63, 64, 65, 127, 129, 257, 385], seed=12)
    sp = SamplingParams(max_tokens=16)
    arrivals = [0, 0, 2, 4, 8, 12, 16, 20]
    alone = [engine(tiny_dirs["C"], dtype_name, num_pages=8, page_size=64, max_num_seqs=1, graphs=False).generate([p], sp)[0]
             for p in ps]
    for pages, graphs in ((128, True), (32, False), (14, True)):
        e = engine(tiny_dirs["C"], dtype_name, num_pages=pages, page_size=64, max_num_seqs=4, max_num_batched_tokens=128,
                   graphs=graphs)
        outs = e.generate(ps, sp, arrival_steps=arrivals)
        assert outs == alone, (pages, graphs)
        assert e.cache.num_requests() == 0 and e.cache.check() == ""


def test_pages_run_out_through_the_engine(tiny_dirs):
    """So few pages that requests are preempted and recomputed: the tokens are still those of a roomy run."""
    from vosti_amd.cache import OutOfPages
    from vosti_amd.sampling import SamplingParams
    ps = prompts("A", [20, 25, 30, 18], seed=6)
    sp = SamplingParams(max_tokens=40)
    roomy = engine(tiny_dirs["A"], "float32", num_pages=64, page_size=8, max_num_seqs=4).generate(ps, sp)
    tight_engine = engine(tiny_dirs["A"], "float32", num_pages=20, page_size=8, max_num_seqs=4)
    assert tight_engine.generate(ps, sp) == roomy and tight_engine.scheduler.preemptions() > 0
    with pytest.raises(OutOfPages):
        engine(tiny_dirs["A"], "float32", num_pages=2, page_size=8).generate([ps[0]], sp)


def test_refusals(tiny_dirs):
    from vosti_amd.sampling import SamplingParams
    e = engine(tiny_dirs["A"], "float32", num_pages=8, page_size=16)
    with pytest.raises(ValueError, match="EmptyPrompt"):
        e.add_request([])
    with pytest.raises(ValueError, match="outside"):
        e.add_request([256])
    with pytest.raises(ValueError, match="HistoryCapacityOverflow"):
        e.add_request([1] * 100, SamplingParams(max_tokens=29))      # 128 positions
    with pytest.raises(ValueError):
        engine(tiny_dirs["A"], "float32", num_pages=8, page_size=12)      # not a power of two


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_command_line(tiny_dirs, tmp_path, dtype_name):
    """The launcher with the reference's environment variables; output as the reference prints it."""
    p = prompts("A", [9], seed=8)[0]
    env = dict(os.environ, MODEL_PATH=str(tiny_dirs["A"]), VOSTI_PROMPT_IDS=",".join(map(str, p)), VOSTI_MAX_TOKENS="5",
               VOSTI_NUM_BLOCKS="4", VOSTI_DTYPE=dtype_name, VOSTI_OUTPUT_TOKENS=str(tmp_path / "out.tsv"),
               VOSTI_ENGINE_STEP_TRACE=str(tmp_path / "trace.jsonl"), PYTHONPATH=str(ROOT))
    r = subprocess.run([sys.executable, "-m", "vosti_amd.launch", "--kind", "engine", "--family", "qwen3"], env=env,
                       capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr[-2000:]
    line = [l for l in r.stdout.splitlines() if l.startswith("MODEL_OUTPUT_TOKEN_IDS=")][0]
    out = json.loads(line.split("=", 1)[1])
    check_greedy_against_plain(PlainQwen3(tiny_dirs["A"], DTYPES[dtype_name]), p, out, dtype_name,
                               PlainQwen3(tiny_dirs["A"], torch.float32))
    assert (tmp_path / "out.tsv").read_text() == "0\t" + ",".join(map(str, out)) + "\n"
    steps = [json.loads(l) for l in (tmp_path / "trace.jsonl").read_text().splitlines()]
    assert len(steps) == 5 and steps[0]["arrived"] == [0] and steps[-1]["emitted"] == {"0": out[-1]}
    # Prepared requests: MAX_TOKENS <TAB> IDS [<TAB> ARRIVAL_STEP], one BENCH line.
    (tmp_path / "reqs.tsv").write_text("# two requests\n3\t1,2,3\n4\t7,8\t2\n")
    env2 = dict(env, VOSTI_BENCH_INPUT=str(tmp_path / "reqs.tsv"))
    r = subprocess.run([sys.executable, "-m", "vosti_amd.launch", "--kind", "engine", "--family", "qwen3", "--",
                        "--output-tokens", str(tmp_path / "o2.tsv")], env=env2, capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr[-2000:]
    assert "BENCH batch=2 prompt_tokens=5 output_tokens=7" in r.stdout
    assert [len(l.split("\t")[1].split(",")) for l in (tmp_path / "o2.tsv").read_text().splitlines()] == [3, 4]
    # A warm-up workload in the same engine first (examples/support/engine_serving.rs:157-206); the measured
    # requests then find the page that the warm-up left: 16 tokens of the 20 they share.
    shared = ",".join(str(7 + (i * 5) % 200) for i in range(20))
    (tmp_path / "warm.tsv").write_text(f"2\t{shared},5\n")
    (tmp_path / "meas.tsv").write_text(f"2\t{shared},9\n2\t{shared},11,12\n")
    env3 = dict(env, VOSTI_BENCH_INPUT=str(tmp_path / "meas.tsv"), VOSTI_BENCH_WARMUP_INPUT=str(tmp_path / "warm.tsv"),
                VOSTI_NUM_BLOCKS="12", VOSTI_PAGE_SIZE="16", VOSTI_MAX_MODEL_LEN="64")
    r = subprocess.run([sys.executable, "-m", "vosti_amd.launch", "--kind", "engine", "--family", "qwen3"], env=env3,
                       capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr[-2000:]
    assert "WARMUP batch=1 prompt_tokens=21 output_tokens=2" in r.stdout
    assert 'WARMUP_CACHE_STATS {"admitted_requests":1,"requests_with_reuse":0,"reused_prefix_blocks":0}' in r.stdout
    assert 'CACHE_STATS {"admitted_requests":2,"requests_with_reuse":2,"reused_prefix_blocks":2' in r.stdout


def test_logits_digest(tiny_dirs, tmp_path, monkeypatch):
    """VOSTI_LOGITS_DIGEST: the hash of every sampled row; a request's hashes are the same alone and in a batch."""
    from vosti_amd.sampling import SamplingParams
    ps = prompts("B", [11, 30], seed=5)
    sp = SamplingParams(max_tokens=4)
    monkeypatch.setenv("VOSTI_LOGITS_DIGEST", str(tmp_path / "alone.txt"))
    engine(tiny_dirs["B"], "bfloat16", num_pages=16, page_size=8).generate([ps[1]], sp)
    monkeypatch.setenv("VOSTI_LOGITS_DIGEST", str(tmp_path / "both.txt"))
    engine(tiny_dirs["B"], "bfloat16", num_pages=16, page_size=8).generate(ps, sp)
    alone = [l.split() for l in (tmp_path / "alone.txt").read_text().splitlines()]
    both = [l.split() for l in (tmp_path / "both.txt").read_text().splitlines()]
    assert len(alone) == 4 and len(both) == 8 and all(len(h) == 64 for _, h in both)
    assert [h for i, h in both if i == "1"] == [h for _, h in alone]


def test_logits_observer_and_multi_call_driver(tiny_dirs, tmp_path):
    """VOSTI_BENCH_CALLS: several calls through one engine, the second built from the first's output
    (examples/support/engine_calls.rs); VOSTI_LOGITS_OBSERVER_DIR: every sampled row as a float32 .npy
    with an index line that carries its hash, its step and the call it belongs to."""
    import numpy as np
    p = prompts("A", [20], seed=8)[0]
    calls = {"prefix_caching": True, "calls": [
        {"label": "first", "prompts": [p], "max_tokens": 3},
        {"label": "second", "max_tokens": 2, "output_prefix_from": {"call": 0, "request": 0, "count": 2, "suffix": [7]}}]}
    (tmp_path / "calls.json").write_text(json.dumps(calls))
    env = dict(os.environ, MODEL_PATH=str(tiny_dirs["A"]), VOSTI_BENCH_CALLS=str(tmp_path / "calls.json"),
               VOSTI_BENCH_CALL_RESULTS=str(tmp_path / "results.json"), VOSTI_LOGITS_OBSERVER_DIR=str(tmp_path / "obs"),
               VOSTI_NUM_BLOCKS="8", VOSTI_PAGE_SIZE="16", VOSTI_DTYPE="float32", PYTHONPATH=str(ROOT))
    r = subprocess.run([sys.executable, "-m", "vosti_amd.launch", "--kind", "engine", "--family", "qwen3"], env=env,
                       capture_output=True, text=True, timeout=110)
    assert r.returncode == 0 and "CALLS_FINISHED 2" in r.stdout, r.stderr[-2000:]
    rec = json.loads((tmp_path / "results.json").read_text())
    first, second = rec
    assert first["label"] == "first" and len(first["output_token_ids"][0]) == 3 and second["request_id_base"] == 1
    assert second["input_token_ids"] == [p + first["output_token_ids"][0][:2] + [7]] and len(second["output_token_ids"][0]) == 2
    index = [json.loads(l) for f in sorted((tmp_path / "obs").glob("observer-*.jsonl")) for l in f.read_text().splitlines()]
    assert [r["phase"] for r in index] == ["call-0"] * 3 + ["call-1"] * 2
    plain = PlainQwen3(tiny_dirs["A"], torch.float32)
    for r, ids in zip(index, [p, p + first["output_token_ids"][0][:1], p + first["output_token_ids"][0][:2]]):
        row = np.load(tmp_path / "obs" / r["artifact"])
        assert row.dtype == np.float32 and row.shape == (256,) and r["argmax"] == int(row.argmax()) and r["finite"]
        torch.testing.assert_close(torch.from_numpy(row), plain.logits(ids)[-1], rtol=1e-4, atol=2e-5)
    assert index[0]["argmax"] == first["output_token_ids"][0][0]


def test_smoke_entry():
    sys.path.insert(0, str(ROOT))
    import __graft_entry__
    __graft_entry__.smoke()


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_padded_graphs_equal_eager(tiny_dirs, dtype_name):
    """Seven requests that end one after the other: the decode steps of 7, 6 and 5 rows are replayed from
    graphs of 8 and 6 rows whose other rows are padding (NaN in the unused pages, which a padding row
    reads, stays in its own row).  The tokens are those of eager steps."""
    from vosti_amd.engine.step import row_bucket
    from vosti_amd.sampling import SamplingParams
    assert [row_bucket(n) for n in (5, 6, 7, 8)] == [6, 6, 8, 8]
    ps = prompts("A", [4, 9, 2, 17, 5, 11, 3], seed=31)
    sp = [SamplingParams(max_tokens=12 + 9 * i, temperature=0.5 * (i % 2), seed=i, ignore_eos=True) for i in range(7)]
    kw = dict(num_pages=64, page_size=16, max_num_seqs=7)
    eager = engine(tiny_dirs["A"], dtype_name, **kw).generate(ps, sp)
    e = engine(tiny_dirs["A"], dtype_name, graphs=True, **kw)
    for t in e.runner.pool.entries:            # poison what no request holds yet: a padding row reads page 0
        if hasattr(t, "k"):
            t.k.fill_(float("nan")); t.v.fill_(float("nan"))
    assert e.generate(ps, sp) == eager
    rows = {key[0] for key in e.runner._captured}
    assert all(row_bucket(r) == r for r in rows) and {8, 6} <= rows, rows


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_graph_replay_equals_eager(tiny_dirs, dtype_name):
    """Decode steps replayed from captured graphs give the tokens of eager steps: several replays of
    each graph, with eager prefill steps, arrivals and a growing block table between them."""
    from vosti_amd.sampling import SamplingParams
    ps = prompts("B", [3, 40, 17, 5], seed=12)
    sp = [SamplingParams(max_tokens=60, temperature=0.7 * (i % 2), seed=i) for i in range(4)]
    kw = dict(num_pages=64, page_size=8, max_num_seqs=3)
    eager = engine(tiny_dirs["B"], dtype_name, **kw).generate(ps, sp, arrival_steps=[0, 0, 5, 30])
    e = engine(tiny_dirs["B"], dtype_name, graphs=True, **kw)
    assert e.generate(ps, sp, arrival_steps=[0, 0, 5, 30]) == eager
    st = e.runner.graph_stats
    assert st["captured"] >= 3 and st["replayed"] > 5 * st["captured"]


def test_a_failed_step_is_given_up_and_planned_again(tiny_dirs):
    """A launch that raises in the middle of a run: the step's rows are given up (their pending tokens,
    not their requests), the error reaches the caller, and going on gives the tokens of an undisturbed run."""
    from vosti_amd.sampling import SamplingParams
    ps = prompts("B", [30, 3, 55], seed=21)
    sp = SamplingParams(max_tokens=12)
    kw = dict(num_pages=40, page_size=8, max_num_seqs=3, max_num_batched_tokens=32)
    want = engine(tiny_dirs["B"], "float32", **kw).generate(ps, sp)
    e = engine(tiny_dirs["B"], "float32", **kw)
    ids = [e.add_request(p, sp) for p in ps]
    outs = {i: [] for i in ids}
    real_run, real_sample = e.runner.run, e.kernels.sample
    steps = 0
    while e.has_unfinished():
        if steps in (1, 4):                     # a forward pass that fails (a prompt step, then a decode step)
            def boom(entries):
                raise RuntimeError("launch failed")
            e.runner.run = boom
        if steps == 6:                          # a sampler that fails after the forward pass ran
            e.kernels.sample = lambda *a, **k: (_ for _ in ()).throw(RuntimeError("sampler failed"))
        try:
            for rid, tok in e.step().items():
                outs[rid].append(tok)
        except RuntimeError as err:
            assert "failed" in str(err)
            assert all(e.cache.pending(r) == 0 for r in ids if e.cache.has_request(r)) and e.cache.check() == ""
        e.runner.run, e.kernels.sample = real_run, real_sample
        steps += 1
        assert steps < 200
    assert [outs[i] for i in ids] == want and e.cache.num_requests() == 0 and e.cache.check() == ""


def test_graphs_are_bounded_and_a_failure_switches_them_off(tiny_dirs):
    from vosti_amd.engine.step import GraphError
    from vosti_amd.sampling import SamplingParams
    ps = prompts("B", [3, 40, 17, 5], seed=12)
    sp = [SamplingParams(max_tokens=60, temperature=0.7 * (i % 2), seed=i) for i in range(4)]
    kw = dict(num_pages=64, page_size=8, max_num_seqs=3)
    eager = engine(tiny_dirs["B"], "bfloat16", **kw).generate(ps, sp, arrival_steps=[0, 0, 5, 30])
    # Two graphs at most: the run needs more signatures than that, so some are captured again after
    # they were dropped; the tokens do not change.
    e = engine(tiny_dirs["B"], "bfloat16", graphs=True, **kw)
    e.runner.max_graphs = 2
    assert e.generate(ps, sp, arrival_steps=[0, 0, 5, 30]) == eager
    st = e.runner.graph_stats
    assert len(e.runner._captured) <= 2 and st["evicted"] >= 1 and st["captured"] == st["evicted"] + len(e.runner._captured)
    # A capture that fails: the error is reported, the step is given up, and no later step is replayed
    # (python/vosti_kernels/graph_overlay.py:120-124, 173-175).
    e = engine(tiny_dirs["B"], "bfloat16", graphs=True, **kw)
    rid = e.add_request(ps[0], SamplingParams(max_tokens=20))
    e.step(); e.step()                                       # prompt, then the first decode step (eager)
    real = e.model.forward
    e.model.forward = lambda *a, **k: (_ for _ in ()).throw(RuntimeError("launch failed under capture"))
    with pytest.raises(GraphError, match="launch failed under capture"):
        e.step()
    e.model.forward = real
    assert e.cache.pending(rid) == 0
    with pytest.raises(GraphError, match="switched off"):
        e.step()
