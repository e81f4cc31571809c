"""The native engine (vosti_engine) against the Python engine and the plain implementation.

Both engines drive the same kernels, cache manager and scheduler; what differs is everything between:
configuration, weight loading, parts, step layout, graph replay, sampling state.  So the native engine's
tokens must be the Python engine's, token for token, and pass the same checks against the plain
implementation, and its logits bit for bit (every rule that both need is computed in one place)."""
import json
import os
import shutil
import subprocess

import pytest
import torch
from safetensors.torch import load_file, save_file

from conftest import TINY
from plain_qwen3 import PlainQwen3
from test_engine_gpu import DTYPES, check_greedy_against_plain, engine, prompts
from test_model_gpu import plain_logits  # noqa: F401  (a fixture)
from vosti_amd.kernels import build

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def program():
    return str(build.ensure("engine", verbose=False))


def run_native(program, dtype_name, env=None, args=(), expect=0):
    lib = build.ensure({"float32": "f32", "bfloat16": "bf16"}[dtype_name], verbose=False)
    base = {k: v for k, v in os.environ.items() if not k.startswith("VOSTI_") and k != "MODEL_PATH"}
    r = subprocess.run([program, "--family", "qwen3", "--dtype", dtype_name, "--lib-dir", str(lib.parent), *args],
                       env=dict(base, **(env or {})), capture_output=True, text=True, timeout=110)
    assert r.returncode == expect, (r.returncode, r.stderr[-2000:])
    return r


def tsv(path, requests):
    path.write_text("".join(f"{m}\t{','.join(map(str, ids))}\t{a}\n" for m, ids, a in requests))


def read_outputs(path):
    return [[int(t) for t in line.split("\t")[1].split(",")] for line in path.read_text().splitlines()]


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
def test_one_prompt_through_the_environment(program, tiny_dirs, tmp_path, name, dtype_name):
    """The reference's way of calling its engine example: everything through environment variables."""
    from vosti_amd.sampling import SamplingParams
    p = prompts(name, [37], seed=5)[0]
    page = TINY[name][1]
    env = dict(MODEL_PATH=str(tiny_dirs[name]), VOSTI_PROMPT_IDS=",".join(map(str, p)), VOSTI_MAX_TOKENS="12",
               VOSTI_NUM_BLOCKS="6", VOSTI_PAGE_SIZE=str(page), VOSTI_OUTPUT_TOKENS=str(tmp_path / "out.tsv"),
               VOSTI_ENGINE_STEP_TRACE=str(tmp_path / "trace.jsonl"))
    r = run_native(program, dtype_name, env)
    line = [l for l in r.stdout.splitlines() if l.startswith("MODEL_OUTPUT_TOKEN_IDS=")][0]
    out = json.loads(line.split("=", 1)[1])
    assert len(out) == 12
    check_greedy_against_plain(PlainQwen3(tiny_dirs[name], DTYPES[dtype_name]), p, out, dtype_name,
                               PlainQwen3(tiny_dirs[name], torch.float32))
    assert read_outputs(tmp_path / "out.tsv") == [out]
    # The Python engine, told the same: the same tokens and the same step trace.
    trace = tmp_path / "py.jsonl"
    with open(trace, "w") as f:
        py = engine(tiny_dirs[name], dtype_name, num_pages=6, page_size=page, max_num_seqs=1).generate(
            [p], SamplingParams(max_tokens=12), trace=f)
    assert py == [out]
    assert [json.loads(l) for l in (tmp_path / "trace.jsonl").read_text().splitlines()] == [json.loads(l) for l in trace.read_text().splitlines()]


@pytest.mark.parametrize("graphs", [0, 1])
@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_staggered_workload_with_temperature(program, tiny_dirs, tmp_path, dtype_name, graphs):
    """Six requests with prompts of 2 to 120 tokens that arrive at different steps, temperature 0.8 with a
    seed each, three rows a step, 48 tokens a step and few pages: prompts are cut into portions, requests
    wait, pages are used again, and (graphs 1) decode steps are replayed from recordings with padding rows.
    Tokens, cache statistics and graph counts are the Python engine's under the same settings."""
    from vosti_amd.sampling import SamplingParams
    ps = prompts("B", [2, 120, 31, 64, 9, 77])
    arrivals = [0, 0, 2, 4, 8, 12]
    tsv(tmp_path / "reqs.tsv", [(24, p, a) for p, a in zip(ps, arrivals)])
    r = run_native(program, dtype_name, args=["--model-path", str(tiny_dirs["B"]), "--bench-input", str(tmp_path / "reqs.tsv"),
                                              "--output-tokens", str(tmp_path / "out.tsv"), "--num-blocks", "40", "--page-size", "8",
                                              "--max-seqs", "3", "--max-batched-tokens", "48", "--temperature", "0.8", "--seed", "100",
                                              "--graphs", str(graphs)])
    outs = read_outputs(tmp_path / "out.tsv")
    assert [len(o) for o in outs] == [24] * 6
    e = engine(tiny_dirs["B"], dtype_name, num_pages=40, page_size=8, max_num_seqs=3, max_num_batched_tokens=48, graphs=bool(graphs))
    params = [SamplingParams(max_tokens=24, temperature=0.8, seed=100 + i) for i in range(6)]
    assert e.generate(ps, params, arrival_steps=arrivals) == outs
    assert f"BENCH batch=6 prompt_tokens={sum(map(len, ps))} output_tokens=144" in r.stdout
    stats = json.loads([l for l in r.stdout.splitlines() if l.startswith("CACHE_STATS ")][0].split(" ", 1)[1])
    assert stats == {"admitted_requests": 6, "requests_with_reuse": e.cache.prefix_hit_requests(),
                     "reused_prefix_blocks": e.cache.prefix_hits(), "preemptions": e.scheduler.preemptions()}
    if graphs:
        g = json.loads([l for l in r.stdout.splitlines() if l.startswith("GRAPH_STATS ")][0].split(" ", 1)[1])
        assert g == e.runner.graph_stats and g["captured"] >= 2 and g["replayed"] > g["captured"]


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_shared_prefixes_end_tokens_and_stored_types(program, tiny_dirs, tmp_path, dtype_name):
    """A folder whose tensors are stored in the other float type than the one computed in (so every tensor
    is converted while loading), with end tokens in generation_config.json; requests that share a prefix
    find each other's pages."""
    from vosti_amd.sampling import SamplingParams
    d = tmp_path / "model"
    shutil.copytree(tiny_dirs["A"], d)
    stored = torch.float32 if dtype_name == "bfloat16" else torch.bfloat16
    t = load_file(str(d / "model.safetensors"))
    save_file({n: (v.to(stored) if n != "model.norm.weight" else v.float()) for n, v in t.items()}, str(d / "model.safetensors"))
    shared = prompts("A", [40], seed=9)[0]
    ps = [shared + [5], shared + [9, 11], shared[:20] + [3]]
    free = engine(d, dtype_name, num_pages=16, page_size=16, max_num_seqs=3).generate(ps, SamplingParams(max_tokens=10))
    eos = sorted({free[0][4], free[1][6]})            # tokens that requests 0 and 1 emit on their way
    (d / "generation_config.json").write_text(json.dumps({"eos_token_id": eos}))
    tsv(tmp_path / "reqs.tsv", [(10, p, a) for p, a in zip(ps, [0, 3, 3])])
    r = run_native(program, dtype_name, args=["--model-path", str(d), "--bench-input", str(tmp_path / "reqs.tsv"), "--num-blocks", "16",
                                              "--page-size", "16", "--output-tokens", str(tmp_path / "out.tsv")])
    outs = read_outputs(tmp_path / "out.tsv")
    e = engine(d, dtype_name, num_pages=16, page_size=16, max_num_seqs=3)
    py = e.generate(ps, SamplingParams(max_tokens=10, eos_token_ids=tuple(eos)), arrival_steps=[0, 3, 3])
    assert outs == py and len(outs[0]) < 10 and outs[0][-1] in eos
    assert f'"requests_with_reuse":{e.cache.prefix_hit_requests()},"reused_prefix_blocks":{e.cache.prefix_hits()}' in r.stdout
    assert e.cache.prefix_hits() >= 3
    # --ignore-eos: to the end of the budget again.
    run_native(program, dtype_name, args=["--model-path", str(d), "--bench-input", str(tmp_path / "reqs.tsv"), "--num-blocks", "16",
                                          "--page-size", "16", "--output-tokens", str(tmp_path / "out2.tsv"), "--ignore-eos"])
    assert read_outputs(tmp_path / "out2.tsv") == engine(d, dtype_name, num_pages=16, page_size=16, max_num_seqs=3).generate(
        ps, SamplingParams(max_tokens=10, eos_token_ids=tuple(eos), ignore_eos=True), arrival_steps=[0, 3, 3])


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_random_weights_are_the_python_package_s(program, tmp_path, dtype_name):
    """--random-weights SEED draws on the GPU what the random-model kind of the Python launcher writes for
    that seed: a folder with nothing but config.json generates the tokens of the written folder.  One line
    per engine step goes to --step-times."""
    from vosti_amd.config import Qwen3Config
    from vosti_amd.sampling import SamplingParams
    from vosti_amd.weights import write_random_model
    cfg = Qwen3Config(**TINY["B"][0])
    written = write_random_model(cfg, 77, tmp_path / "written", DTYPES[dtype_name])
    bare = tmp_path / "bare"
    bare.mkdir()
    shutil.copy(written / "config.json", bare / "config.json")
    p = prompts("B", [50], seed=2)[0]
    r = run_native(program, dtype_name, args=["--model-path", str(bare), "--random-weights", "77", "--prompt-ids", ",".join(map(str, p)),
                                              "--max-tokens", "10", "--num-blocks", "16", "--page-size", "8", "--step-times", str(tmp_path / "times.txt")])
    out = json.loads([l for l in r.stdout.splitlines() if l.startswith("MODEL_OUTPUT_TOKEN_IDS=")][0].split("=", 1)[1])
    assert [out] == engine(written, dtype_name, num_pages=16, page_size=8, max_num_seqs=1).generate([p], SamplingParams(max_tokens=10))
    times = [l.split() for l in (tmp_path / "times.txt").read_text().splitlines()]
    assert [(int(t[0]), int(t[1]), int(t[2])) for t in times] == [(1, 50, 1)] + [(1, 1, 1)] * 9 and all(float(t[3]) > 0 for t in times)


@pytest.mark.parametrize("graphs", [False, True])
@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_native_engine_from_python(tiny_dirs, dtype_name, graphs):
    """NativeEngine is the native engine behind Engine's face: the same requests, the same tokens, in one
    process with the Python engine (one HIP runtime, one kernel library, streams of their own)."""
    from vosti_amd.engine import NativeEngine, NativeEngineError
    from vosti_amd.sampling import SamplingParams
    ps = prompts("A", [4, 9, 2, 17, 5, 11, 3], seed=31)
    sp = [SamplingParams(max_tokens=12 + 9 * i, temperature=0.5 * (i % 2), seed=i, ignore_eos=True) for i in range(7)]
    kw = dict(num_pages=64, page_size=16, max_num_seqs=7, graphs=graphs)
    want = engine(tiny_dirs["A"], dtype_name, **kw).generate(ps, sp, arrival_steps=[0, 0, 1, 1, 2, 5, 9])
    native = NativeEngine(tiny_dirs["A"], dtype=dtype_name, **kw)
    assert native.generate(ps, sp, arrival_steps=[0, 0, 1, 1, 2, 5, 9]) == want
    st = native.stats()
    assert st["cache_requests"] == 0 and native.cache_check() == "" and not native.has_unfinished()
    assert (st["graph_stats"]["replayed"] > 0) == graphs
    # Step by step, and what it refuses.
    rid = native.add_request(ps[2], SamplingParams(max_tokens=3))        # a greedy one
    got = []
    while native.has_unfinished():
        got += [t for r, t in native.step().items() if r == rid]
    assert got == want[2][:3]
    with pytest.raises(ValueError, match="EmptyPrompt"):
        native.add_request([], SamplingParams(max_tokens=3))
    with pytest.raises(ValueError, match="prompt token outside"):
        native.add_request([10 ** 6], SamplingParams(max_tokens=3))
    with pytest.raises(NativeEngineError, match="config.json is missing"):
        NativeEngine("/nonexistent", dtype=dtype_name)


def test_workspace_asked_for_twice_in_one_forward(tmp_path):
    """A step that is not replayed from a recording, in which the attention asks for the step's workspace twice
    and for more the second time: 20 decoded rows over 2,310 keys need more floats of partial results than
    the qkv projection's chunk sums took, and the output projection after them goes through chunk sums again
    (matrices large enough for that route: 6144 x 2048 and 2048 x 4096).  The buffer of the first request must
    outlive the second; the tokens are the Python engine's."""
    import random
    from vosti_amd.config import Qwen3Config
    from vosti_amd.engine import NativeEngine
    from vosti_amd.kernels.ops import SEGMENT_KEYS, kernels_for
    from vosti_amd.sampling import SamplingParams
    from vosti_amd.weights import write_random_model
    cfg = Qwen3Config(vocab_size=1000, hidden_size=2048, intermediate_size=512, num_hidden_layers=1, num_attention_heads=32,
                      num_key_value_heads=8, head_dim=128, max_position_embeddings=4096, rms_norm_eps=1e-6, rope_theta=1e6,
                      tie_word_embeddings=False)
    write_random_model(cfg, 3, tmp_path)
    k = kernels_for("bfloat16")
    rows, keys = 20, 2310
    chunk_sums = k.gemm_workspace_floats(rows, (32 + 2 * 8) * 128, 2048)
    assert 0 < chunk_sums < k.attn_scratch_floats(rows, 32, 128, -(-keys // SEGMENT_KEYS)) and k.gemm_workspace_floats(rows, 2048, 32 * 128) > 0
    rng = random.Random(2)
    ps = [[rng.randrange(1000) for _ in range(keys)] for _ in range(rows)]
    kw = dict(num_pages=rows * 37 + 8, page_size=64, max_num_seqs=rows, max_num_batched_tokens=8192, graphs=False)
    sp = SamplingParams(max_tokens=3, ignore_eos=True)
    want = engine(tmp_path, "bfloat16", **kw).generate(ps, sp)
    assert NativeEngine(tmp_path, dtype="bfloat16", **kw).generate(ps, sp) == want


@pytest.mark.parametrize("dtype_name", ["bfloat16", "float32"])
def test_busy_workload_at_the_measured_width(tmp_path, dtype_name):
    """Two layers of the measured model's width, 40 requests: prompts of 20 to 1,500 tokens, half of them behind
    a shared prefix of 300 tokens, 8 to 70 new tokens each, a third at a temperature, arriving over 30 steps,
    at most 24 rows and 1,024 tokens a step and a third of the pages they would need together: prompts in
    portions beside decoding rows, prefix pages found and evicted, requests taken back and computed again,
    decode steps of 1 to 24 rows replayed from recordings with padding.  Every kernel runs at the sizes of the
    measurements (17 to 64 rows through chunk sums among them) on memory that the native engine allocates
    tensor by tensor.  Tokens and statistics are the Python engine's."""
    import random
    from vosti_amd.config import Qwen3Config
    from vosti_amd.engine import NativeEngine
    from vosti_amd.sampling import SamplingParams
    from vosti_amd.weights import write_random_model
    V = 4999
    cfg = Qwen3Config(vocab_size=V, hidden_size=4096, intermediate_size=12288, num_hidden_layers=2, num_attention_heads=32,
                      num_key_value_heads=8, head_dim=128, max_position_embeddings=4096, rms_norm_eps=1e-6, rope_theta=1e6,
                      tie_word_embeddings=False)
    write_random_model(cfg, 11, tmp_path)
    rng = random.Random(5)
    shared = [rng.randrange(V) for _ in range(300)]
    ps, sp, arrivals = [], [], []
    for i in range(40):
        own = [rng.randrange(V) for _ in range(rng.choice((20, 70, 200, 450, 900, 1500)))]
        ps.append(shared + own if i % 2 else own)
        sp.append(SamplingParams(max_tokens=rng.randrange(8, 71), temperature=0.7 if i % 3 == 0 else 0.0, seed=i, ignore_eos=True))
        arrivals.append(rng.randrange(0, 30))
    need = sum(-(-(len(p) + s.max_tokens) // 64) for p, s in zip(ps, sp))
    kw = dict(num_pages=need // 3, page_size=64, max_num_seqs=24, max_num_batched_tokens=1024, graphs=True, enable_prefix_cache=True)
    e = engine(tmp_path, dtype_name, **kw)
    want = e.generate(ps, sp, arrival_steps=arrivals)
    assert [len(o) for o in want] == [s.max_tokens for s in sp]
    native = NativeEngine(tmp_path, dtype=dtype_name, **kw)
    assert native.generate(ps, sp, arrival_steps=arrivals) == want
    st = native.stats()
    assert st["preemptions"] == e.scheduler.preemptions() and st["prefix_hits"] == e.cache.prefix_hits() > 0
    assert st["graph_stats"] == e.runner.graph_stats and st["graph_stats"]["replayed"] > 20
    assert st["cache_requests"] == 0 and native.cache_check() == ""


class _NativeRunner:
    """The native engine's step function behind the face that test_model_gpu's replay() drives."""

    class _Cache:
        def __init__(self, engine):
            self.engine = engine

        def num_requests(self):
            return self.engine.stats()["cache_requests"]

        def check(self):
            return self.engine.cache_check()

    class _Identity:
        @staticmethod
        def to_f32(x):
            return x

    def __init__(self, model_dir, dtype_name, page_size, num_pages):
        from vosti_amd.engine import NativeEngine
        self.engine = NativeEngine(model_dir, dtype=dtype_name, num_pages=num_pages, page_size=page_size, max_num_seqs=8,
                                   enable_prefix_cache=False, graphs=False)
        self.cache, self.kernels = self._Cache(self.engine), self._Identity()

    def step(self, entries):
        return torch.from_numpy(self.engine.trace_step([(e.request_id, e.tokens, e.want) for e in entries]))

    def finish(self, rid):
        self.engine.trace_finish(rid)


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_every_cutting_through_the_native_step_function(tiny_dirs, plain_logits, name, dtype_name):
    """The native engine's step function under the four cuttings of the Python one's test: every request alone
    and whole; all but the last 32 tokens in one step and the rest one by one; portions of changing size down to
    one token; up to four live requests mixed, on so few pages that they are used again.  The whole prompts'
    logits are the plain implementation's within what the type costs, the logits of every (request, position)
    are the same bits under all four cuttings, and they are the bits of the Python step function."""
    from test_model_gpu import (LENGTHS, assert_matches_plain, cut_chunks, cut_mixed, cut_tail, cut_whole, make_runner, prompts_for,
                                replay)
    prompts = prompts_for(name)
    page = TINY[name][1]
    ref, exact = plain_logits(name, dtype_name), plain_logits(name, "float32")
    mixed_steps, mixed_pages = cut_mixed(prompts, page)
    pages = -(-max(LENGTHS[name]) // page)
    runner = _NativeRunner(tiny_dirs[name], dtype_name, page, pages)
    whole = replay(runner, cut_whole(prompts))
    for i, p in enumerate(prompts):
        got = torch.stack([whole[(i, j)] for j in range(len(p))])
        assert_matches_plain(got, ref[i], exact[i], dtype_name, f"request {i} (length {len(p)}), whole, native step function")
    for label, steps, n in (("tail", cut_tail(prompts), None), ("chunks", cut_chunks(prompts), None), ("mixed", mixed_steps, mixed_pages)):
        if n is not None:
            runner = _NativeRunner(tiny_dirs[name], dtype_name, page, n)
        got = replay(runner, steps)
        assert set(got) == set(whole), label
        bad = [k for k in sorted(whole) if not torch.equal(got[k], whole[k])]
        assert not bad, f"{label}: first differing (request, position) {bad[:1]} of {len(bad)}"
    py = replay(make_runner(tiny_dirs[name], dtype_name, page, num_pages=pages), cut_whole(prompts))
    differing = [k for k in sorted(whole) if not torch.equal(py[k], whole[k])]
    assert not differing, f"the two step functions differ at {differing[:1]} and {len(differing) - 1} more places"


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_replayed_steps_through_the_step_function_alone(tiny_dirs, dtype_name):
    """The step function alone with recorded decode steps: four requests decode together (eagerly, recorded, then
    replayed), and between the replays one of them decodes alone, a step that runs eagerly and leaves the
    activation memory's cursor far below the recording's results.  The 32-bit copy of a replayed step's logits
    must not be placed on top of them: every step's logits are those of an engine that replays nothing."""
    from vosti_amd.engine import NativeEngine
    ps = prompts("B", [9, 30, 17, 5], seed=12)
    got = {}
    for graphs in (False, True):
        e = NativeEngine(tiny_dirs["B"], dtype=dtype_name, num_pages=64, page_size=8, max_num_seqs=8, enable_prefix_cache=False, graphs=graphs)
        out = [e.trace_step([(i, p, [len(p) - 1]) for i, p in enumerate(ps)])]
        tok = 7
        for round_ in range(4):
            for _ in range(3):                                       # all four rows: eager, recorded, replayed, ...
                out.append(e.trace_step([(i, [tok + i], [0]) for i in range(4)]))
                tok += 4
            alone = round_ % 4
            out.append(e.trace_step([(alone, [tok], [0])]))          # fewer rows, eagerly at first sight
            tok += 1
        if graphs:
            assert e.stats()["graph_stats"]["replayed"] >= 8
        for i in range(4):
            e.trace_finish(i)
        assert e.cache_check() == ""
        got[graphs] = out
    for a, b in zip(got[False], got[True]):
        assert a.shape == b.shape and (a.view("<u4") == b.view("<u4")).all()


FAMILY_WIDTHS = {       # hidden, inside, q heads, kv heads (head size 128): the layer sizes of the family's models
    "0.6b": (1024, 3072, 16, 8), "1.7b": (2048, 6144, 16, 8), "4b": (2560, 9728, 32, 8), "14b": (5120, 17408, 40, 8), "32b": (5120, 25600, 64, 8),
}


@pytest.mark.parametrize("shape", sorted(FAMILY_WIDTHS))
def test_the_family_s_other_widths_through_both_engines(tmp_path, shape):
    """One layer of each of the family's other layer sizes (the projections then take other kernels: two to twelve
    waves a workgroup in the streaming kernels, the route through chunk sums at other row counts, other tile
    grids) under a small staggered workload with recorded decode steps of 1 to 20 rows and prompts in portions:
    the native engine's tokens are the Python engine's, and the first request's are the plain implementation's
    choices within the type's cost."""
    import random
    from vosti_amd.config import Qwen3Config
    from vosti_amd.engine import NativeEngine
    from vosti_amd.sampling import SamplingParams
    from vosti_amd.weights import write_random_model
    H, I, nq, nkv = FAMILY_WIDTHS[shape]
    V = 2003
    cfg = Qwen3Config(vocab_size=V, hidden_size=H, intermediate_size=I, num_hidden_layers=1, num_attention_heads=nq,
                      num_key_value_heads=nkv, head_dim=128, max_position_embeddings=2048, rms_norm_eps=1e-6, rope_theta=1e6,
                      tie_word_embeddings=H <= 2560)
    write_random_model(cfg, 21, tmp_path)
    rng = random.Random(len(shape) + H)
    ps = [[rng.randrange(V) for _ in range(rng.choice((5, 40, 130, 300, 700)))] for _ in range(20)]
    sp = [SamplingParams(max_tokens=rng.randrange(6, 30), temperature=0.6 if i % 4 == 1 else 0.0, seed=i, ignore_eos=True) for i in range(20)]
    arrivals = [rng.randrange(0, 12) for _ in ps]
    kw = dict(num_pages=20 * 12, page_size=64, max_num_seqs=20, max_num_batched_tokens=512, graphs=True)
    e = engine(tmp_path, "bfloat16", **kw)
    want = e.generate(ps, sp, arrival_steps=arrivals)
    native = NativeEngine(tmp_path, dtype="bfloat16", **kw)
    assert native.generate(ps, sp, arrival_steps=arrivals) == want
    assert native.stats()["graph_stats"] == e.runner.graph_stats and native.cache_check() == ""
    first = next(i for i in range(20) if sp[i].temperature == 0.0 and len(ps[i]) <= 130)
    check_greedy_against_plain(PlainQwen3(tmp_path, torch.bfloat16), ps[first], want[first], "bfloat16", PlainQwen3(tmp_path, torch.float32))


def test_python_launcher_with_the_native_engine(tiny_dirs, tmp_path):
    """--engine native of the Python launcher prints what --engine python prints (but for the wall time)."""
    import sys
    from conftest import ROOT
    ps = prompts("B", [30, 30, 12], seed=4)
    ps[1] = ps[0][:24] + ps[1][24:]                    # shares three pages of 8 with the first
    tsv(tmp_path / "reqs.tsv", [(6, p, a) for p, a in zip(ps, [0, 2, 2])])
    lines = {}
    for which in ("python", "native"):
        r = subprocess.run([sys.executable, "-m", "vosti_amd.launch", "--kind", "engine", "--family", "qwen3", "--", "--engine", which,
                            "--model-path", str(tiny_dirs["B"]), "--bench-input", str(tmp_path / "reqs.tsv"), "--page-size", "8",
                            "--num-blocks", "24", "--graphs", "1", "--output-tokens", str(tmp_path / f"{which}.tsv")],
                           env=dict(os.environ, PYTHONPATH=str(ROOT)), capture_output=True, text=True, timeout=110)
        assert r.returncode == 0, r.stderr[-2000:]
        lines[which] = [l.split(" wall_s=")[0] for l in r.stdout.splitlines() if l.split(" ")[0] in ("BENCH", "CACHE_STATS", "GRAPH_STATS")]
    assert lines["native"] == lines["python"] and len(lines["native"]) == 3
    assert (tmp_path / "native.tsv").read_text() == (tmp_path / "python.tsv").read_text()
    assert '"reused_prefix_blocks":3' in lines["native"][1]


def test_one_error_for_weights_that_do_not_fit(program, tiny_dirs, tmp_path):
    d = tmp_path / "model"
    shutil.copytree(tiny_dirs["B"], d)
    t = load_file(str(d / "model.safetensors"))
    del t["model.layers.1.mlp.up_proj.weight"]
    t["model.layers.0.self_attn.q_norm.weight"] = torch.ones(8)
    t["model.layers.7.extra"] = torch.zeros(2)
    save_file(t, str(d / "model.safetensors"))
    r = run_native(program, "bfloat16", args=["--model-path", str(d)], expect=1)
    assert "missing (1): model.layers.1.mlp.up_proj.weight" in r.stderr
    assert "unexpected (1): model.layers.7.extra" in r.stderr
    assert "wrong shape or type (1): model.layers.0.self_attn.q_norm.weight: file has [8], model needs [32]" in r.stderr
    # Pages that cannot hold the request: refused, not run.
    r = run_native(program, "bfloat16", args=["--model-path", str(tiny_dirs["B"]), "--prompt-ids", ",".join(["7"] * 100),
                                              "--num-blocks", "2", "--page-size", "8"], expect=1)
    assert "more cache pages than the pool has" in r.stderr
