"""The engine against the plain implementation, under every way of cutting the work."""
import json
import os
import random
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

from conftest import ROOT, TINY
from plain_qwen3 import PlainQwen3

pytestmark = pytest.mark.gpu

DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
# float32: only summation order and the last bit of exp / rsqrt differ.
TOL = {"float32": dict(rtol=1e-4, atol=2e-5)}


def assert_matches_plain(got, ref, exact, dtype_name, what=""):
    """got: the engine's logits; ref: the plain implementation's in the same type; exact: the plain
    implementation's in float32.  In float32 a tolerance.  In bfloat16 the plain implementation rounds
    where the engine does, but a sum taken in another order can land on the neighbouring value and the
    layers carry that on, so a fixed tolerance is either loose or wrong: the measure is what the type
    itself costs.  On average the engine must lie closer to the plain bfloat16 logits than those lie to
    the plain float32 logits.  At the worst element it may be off by twice the type's worst cost: where
    the two differ, a value has landed on the neighbouring one, a whole step of the type, which is twice
    the largest error that a rounding makes.  (Measured on the tiny models: 0.006 to 0.008 at the worst
    element, one step of a logit between 1 and 2, against a worst cost of 0.005 to 0.006; 0.0001 to 0.0007
    on average against 0.0006 to 0.001.)  A rounding point the engine misses (P before P.V, the tables,
    a norm fed the rounded residual) costs about as much as the type does, and a fault of indexing or
    masking a hundred times more."""
    if dtype_name == "float32":
        torch.testing.assert_close(got, ref, **TOL["float32"], msg=lambda m: f"{what}: {m}")
        return
    assert got.shape == ref.shape == exact.shape
    cost, dev = (ref - exact).abs(), (got - ref).abs()
    assert dev.max() <= 2 * cost.max() and dev.mean() <= cost.mean(), \
        f"{what}: deviation max {dev.max():.5f} mean {dev.mean():.6f}, the type's cost max {cost.max():.5f} mean {cost.mean():.6f}"
LENGTHS = {"A": [1, 7, 33, 64, 100, 128], "B": [2, 17, 63, 65, 120, 129, 200, 256], "C": [3, 64, 65, 130, 257, 300, 512]}


def prompts_for(name):
    rng = random.Random(ord(name) + 11)
    vocab = TINY[name][0]["vocab_size"]
    return [[rng.randrange(vocab) for _ in range(n)] for n in LENGTHS[name]]


@pytest.fixture(scope="module")
def plain_logits(tiny_dirs):
    """Plain logits of every prompt, per configuration and type, computed once."""
    cache = {}

    def get(name, dtype_name):
        key = (name, dtype_name)
        if key not in cache:
            model = PlainQwen3(tiny_dirs[name], DTYPES[dtype_name])
            cache[key] = [model.logits(p) for p in prompts_for(name)]
        return cache[key]
    return get


def make_runner(model_dir, dtype_name, page_size, num_pages, num_slots=8):
    from vosti_amd.cache import CachePool
    from vosti_amd.engine import ModelRunner
    from vosti_amd.models import load_model
    model = load_model(model_dir, dtype_name)
    return ModelRunner(model, CachePool(model, page_size=page_size, num_pages=num_pages, num_slots=num_slots))


def replay(runner, steps):
    """steps: list of (entries [(rid, tokens, want)], end [rid]) -> {(rid, position): float32 logits row}."""
    from vosti_amd.engine import StepEntry
    out, fed = {}, {}
    for entries, end in steps:
        logits = runner.kernels.to_f32(runner.step([StepEntry(r, t, w) for r, t, w in entries])).cpu()
        row = 0
        for r, t, w in entries:
            base = fed.get(r, 0)
            for place in w:
                out[(r, base + place)] = logits[row]
                row += 1
            fed[r] = base + len(t)
        for r in end:
            runner.finish(r)
            fed.pop(r, None)
    assert runner.cache.num_requests() == 0 and runner.cache.check() == ""
    return out


def cut_whole(prompts):
    return [([(i, p, list(range(len(p))))], [i]) for i, p in enumerate(prompts)]


def cut_tail(prompts, tail=32):
    steps = []
    for i, p in enumerate(prompts):
        head = max(1, len(p) - tail)
        steps.append(([(i, p[:head], list(range(head)))], []))
        for j in range(head, len(p)):
            steps.append(([(i, p[j:j + 1], [0])], []))
        steps[-1][1].append(i)
    return steps


def cut_chunks(prompts, sizes=(7, 2, 33, 16, 5, 2, 64, 3, 1, 31)):
    steps, k = [], 0
    for i, p in enumerate(prompts):
        pos = 0
        while pos < len(p):
            n = min(sizes[k % len(sizes)], len(p) - pos)
            k += 1
            steps.append(([(i, p[pos:pos + n], list(range(n)))], []))
            pos += n
        steps[-1][1].append(i)
    return steps


def cut_mixed(prompts, page, max_live=4, seed=5):
    """Up to four live requests, portions of some beside single tokens of others; returns the
    steps and the pool size (pages) that just holds the largest set of live requests."""
    rng = random.Random(seed)
    order = list(range(len(prompts)))
    rng.shuffle(order)
    waiting, live, pos, steps = order[:], [], {}, []
    peak = 0
    while waiting or live:
        while waiting and len(live) < max_live:
            r = waiting.pop(0)
            live.append(r)
            pos[r] = 0
        peak = max(peak, sum(-(-len(prompts[r]) // page) for r in live))
        entries, end = [], []
        for r in list(live):
            if rng.random() < 0.2 and len(live) > 1:
                continue                       # left out of this step, goes on later
            left = len(prompts[r]) - pos[r]
            n = min(left, rng.choice([1, 1, 1, 2, 3, 9, 16, 40]))
            entries.append((r, prompts[r][pos[r]:pos[r] + n], list(range(n))))
            pos[r] += n
            if pos[r] == len(prompts[r]):
                end.append(r)
                live.remove(r)
        if entries:
            steps.append((entries, end))
    return steps, peak


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_every_cutting(tiny_dirs, plain_logits, name, dtype_name):
    prompts = prompts_for(name)
    page = TINY[name][1]
    ref, exact = plain_logits(name, dtype_name), plain_logits(name, "float32")
    mixed_steps, mixed_pages = cut_mixed(prompts, page)
    runner = make_runner(tiny_dirs[name], dtype_name, page, num_pages=-(-max(LENGTHS[name]) // page))
    whole = replay(runner, cut_whole(prompts))
    for i, p in enumerate(prompts):
        got = torch.stack([whole[(i, j)] for j in range(len(p))])
        assert_matches_plain(got, ref[i], exact[i], dtype_name, f"request {i} (length {len(p)}), whole")
    for label, steps, pages in (("tail", cut_tail(prompts), None), ("chunks", cut_chunks(prompts), None),
                                ("mixed", mixed_steps, mixed_pages)):
        if pages is not None:
            runner = make_runner(tiny_dirs[name], dtype_name, page, num_pages=pages)
        got = replay(runner, steps)
        assert set(got) == set(whole), label
        bad = [k for k in sorted(whole) if not torch.equal(got[k], whole[k])]
        assert not bad, f"{label}: first differing (request, position) {bad[0]} of {len(bad)}; " \
                        f"max diff {(got[bad[0]] - whole[bad[0]]).abs().max().item():.3e}"


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_page_size_64_and_first_tokens(tiny_dirs, plain_logits, dtype_name):
    """The default page size, and the first tokens of a sequence one by one from an empty cache."""
    name = "B"
    prompts = prompts_for(name)
    ref, exact = plain_logits(name, dtype_name), plain_logits(name, "float32")
    runner = make_runner(tiny_dirs[name], dtype_name, 64, num_pages=4)
    i = 7
    steps = [([(0, prompts[i][j:j + 1], [0])], []) for j in range(40)]
    got = replay(runner, steps + [([(0, prompts[i][40:], list(range(len(prompts[i]) - 40)))], [0])])
    stacked = torch.stack([got[(0, j)] for j in range(len(prompts[i]))])
    assert_matches_plain(stacked, ref[i], exact[i], dtype_name, "first tokens one by one")


def test_weights_are_kept_in_their_types(tiny_dirs):
    from vosti_amd.models import load_model
    m = load_model(tiny_dirs["A"], "bfloat16")
    assert m.embedding.weight.dtype == torch.bfloat16 and m.head.weight is m.embedding.weight
    assert m.layers[0].mixer.w_qkv.dtype == torch.bfloat16
    m32 = load_model(tiny_dirs["A"], "float32")
    assert m32.layers[0].mixer.w_qkv.dtype == torch.float32


def run_trace(model_dir, dtype_name, out_dir, max_tokens, steps, page_size=None, extra=()):
    cmd = [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(model_dir), "--dtype", dtype_name, "--out",
           str(out_dir), "--max-tokens", str(max_tokens), *extra]
    if page_size:
        cmd += ["--page-size", str(page_size)]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    for rec in steps:
        proc.stdin.write(json.dumps(rec) + "\n")
        proc.stdin.flush()
        assert proc.stdout.readline().strip() == f"done {rec['step']}"
    proc.stdin.close()
    assert proc.wait(timeout=60) == 0


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_trace_run_program(tiny_dirs, plain_logits, tmp_path, dtype_name):
    """The command-line tool: two requests interleaved, pages for just these two, then a third
    request that can only run on pages the first ones gave back."""
    name = "B"
    prompts = prompts_for(name)
    ref, exact = plain_logits(name, dtype_name), plain_logits(name, "float32")
    a, b, c = 3, 5, 4     # lengths 65, 129, 120
    vocab = TINY[name][0]["vocab_size"]
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": prompts[a][:40], "want": [0, 39]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": prompts[a][40:], "want": [24]},
                                {"id": "b", "tokens": prompts[b][:100], "want": []}], "end": ["a"]},
        {"step": 9, "entries": [], "end": []},                      # a step that brings nothing: answered, no file
        {"step": 2, "entries": [{"id": "b", "tokens": prompts[b][100:128], "want": [27]},
                                {"id": "idle", "tokens": [], "want": []}], "end": ["never seen"]},      # an entry without tokens is as good as left out
        {"step": 3, "entries": [{"id": "b", "tokens": prompts[b][128:], "want": [0]}], "end": ["b"]},
        {"step": 4, "entries": [{"id": "c", "tokens": prompts[c], "want": [119]}], "end": ["c"]},
    ]
    run_trace(tiny_dirs[name], dtype_name, tmp_path, max_tokens=128 + 192, steps=steps)
    assert not (tmp_path / "9.f32").exists()
    read = lambda s, d=tmp_path: torch.from_numpy(np.fromfile(d / f"{s}.f32", dtype="<f4").reshape(-1, vocab))
    # The few rows that were asked for, against the same rows of the plain logits.
    got = torch.cat([read(s) for s in range(5)])
    pick = lambda t: torch.cat([t[a][[0, 39]], t[a][[64]], t[b][[127]], t[b][[128]], t[c][[119]]])
    assert_matches_plain(got, pick(ref), pick(exact), dtype_name, "trace_run")
    # Which row is which: an index beside every step's file.
    index = [json.loads((tmp_path / f"{s}.json").read_text()) for s in range(5)]
    assert [i["rows"] for i in index] == [[["a", 0], ["a", 39]], [["a", 64]], [["b", 127]], [["b", 128]], [["c", 119]]]
    assert all(i["vocab"] == vocab and i["step"] == s for s, i in enumerate(index))
    # That was the native engine's step function (the library has every part of this model).  The same trace
    # through the Python step function, the path of models whose parts exist in Python alone: the same kernels and
    # cache manager under other host code, and every rule both need computed in one place, so the same bits.
    python_dir = tmp_path / "python"
    python_dir.mkdir()
    run_trace(tiny_dirs[name], dtype_name, python_dir, max_tokens=128 + 192, steps=steps, extra=["--engine", "python"])
    assert torch.equal(torch.cat([read(s, python_dir) for s in range(5)]), got)


FULL_WIDTH = dict(vocab_size=4999, hidden_size=4096, intermediate_size=12288, num_hidden_layers=2, num_attention_heads=32,
                  num_key_value_heads=8, head_dim=128, max_position_embeddings=4096, rms_norm_eps=1e-6, rope_theta=1e6,
                  tie_word_embeddings=False)


@pytest.fixture(scope="module")
def full_width_dir(tmp_path_factory):
    from vosti_amd.config import Qwen3Config
    from vosti_amd.weights import write_random_model
    d = tmp_path_factory.mktemp("full_width")
    write_random_model(Qwen3Config(**FULL_WIDTH), 7, d, dtype=torch.bfloat16)
    return d


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_layers_of_full_width(full_width_dir, dtype_name):
    """Two layers with the sizes of the measured model (width 4096, 32 and 8 heads of 128, 12288 inside)
    and a small vocabulary: the kernels that the measurements run (streamed weights with the activation
    resident, gate/up with the activation folded in, the pipelined tile kernel, prompt attention through
    LDS) against the plain implementation, and every cutting against the whole prompts bit for bit.

    In 32-bit the whole prompts meet the plain logits within the tolerance of the tiny models.  In
    bfloat16 sums of 4,096 and 12,288 terms taken in another order land on neighbouring values often
    enough that the tiny models' tolerance is no measure; there the engine must lie closer to the plain
    bfloat16 logits than those lie to the plain 32-bit logits, at the worst element and on average: its
    deviation is then below what the type itself costs, and any fault of indexing or masking is far above."""
    d = full_width_dir
    rng = random.Random(21)
    prompts = [[rng.randrange(FULL_WIDTH["vocab_size"]) for _ in range(n)] for n in (5, 150, 330)]
    runner = make_runner(d, dtype_name, 64, num_pages=6)
    whole = replay(runner, cut_whole(prompts))
    plain = PlainQwen3(d, DTYPES[dtype_name])
    exact = PlainQwen3(d, torch.float32) if dtype_name == "bfloat16" else None
    for i in (0, 1):
        got = torch.stack([whole[(i, j)] for j in range(len(prompts[i]))])
        ref = plain.logits(prompts[i])
        assert_matches_plain(got, ref, exact.logits(prompts[i]) if exact else ref, dtype_name, f"request {i}")
    mixed_steps, mixed_pages = cut_mixed(prompts, 64)
    cuttings = [("tail", cut_tail(prompts), 6), ("chunks", cut_chunks(prompts), 6), ("mixed", mixed_steps, mixed_pages)]
    for label, steps, pages in cuttings if dtype_name == "bfloat16" else cuttings[1:2]:
        got = replay(make_runner(d, dtype_name, 64, num_pages=pages), steps)
        bad = [k for k in sorted(whole) if not torch.equal(got[k], whole[k])]
        assert set(got) == set(whole) and not bad, f"{label}: first differing (request, position) {bad[:1]} of {len(bad)}"


SWEEP = [
    # hidden, layers, q heads, kv heads, head size, inside, vocab, page, eps, theta, tied
    (80, 1, 3, 3, 80, 96, 211, 32, 1e-6, 1e4, True),        # one q head per kv head, head size 80
    (128, 2, 8, 1, 64, 200, 777, 128, 1e-5, 1e6, False),    # eight q heads on one kv head, pages of two tiles
    (512, 1, 6, 2, 128, 520, 300, 64, 1e-6, 5e5, False),    # width of one chunk, groups of three
    (96, 2, 2, 2, 48, 64, 97, 8, 1e-5, 1e5, True),          # head size 48, the smallest page
    (1024, 1, 2, 1, 256, 1032, 130, 64, 1e-6, 1e6, False),  # head size 256, two chunks
]


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", range(len(SWEEP)))
def test_other_shapes(tmp_path_factory, case, dtype_name):
    """Shapes that take other kernels or other branches of them than the tiny configurations do (head
    sizes 48, 80 and 256, groups of 1, 3 and 8 q heads, pages of 8 to 128, widths of one and two chunks):
    whole prompts against the plain implementation, two cuttings against the whole prompts bit for bit."""
    from vosti_amd.config import Qwen3Config
    from vosti_amd.weights import write_random_model
    H, L, nq, nkv, d, I, V, page, eps, theta, tied = SWEEP[case]
    cfg = dict(vocab_size=V, hidden_size=H, intermediate_size=I, num_hidden_layers=L, num_attention_heads=nq,
               num_key_value_heads=nkv, head_dim=d, max_position_embeddings=320, rms_norm_eps=eps, rope_theta=theta,
               tie_word_embeddings=tied)
    folder = tmp_path_factory.mktemp(f"sweep_{case}")
    write_random_model(Qwen3Config(**cfg), 30 + case, folder, dtype=torch.bfloat16)
    rng = random.Random(50 + case)
    prompts = [[rng.randrange(V) for _ in range(n)] for n in (3, 70, 129, 300)]
    plain = PlainQwen3(folder, DTYPES[dtype_name])
    exact = PlainQwen3(folder, torch.float32) if dtype_name == "bfloat16" else plain
    pages = -(-300 // page) + 1
    whole = replay(make_runner(folder, dtype_name, page, num_pages=pages), cut_whole(prompts))
    for i, p in enumerate(prompts):
        got = torch.stack([whole[(i, j)] for j in range(len(p))])
        assert_matches_plain(got, plain.logits(p), exact.logits(p), dtype_name, f"case {case}, request {i}")
    for label, steps in (("tail", cut_tail(prompts)), ("chunks", cut_chunks(prompts))):
        got = replay(make_runner(folder, dtype_name, page, num_pages=pages), steps)
        bad = [k for k in sorted(whole) if not torch.equal(got[k], whole[k])]
        assert set(got) == set(whole) and not bad, f"case {case}, {label}: first differing (request, position) {bad[:1]} of {len(bad)}"


def test_long_context_at_full_width(full_width_dir):
    """A request of 2,400 tokens at the measured model's layer width: decode attention over ten
    segments and their combination, prompt portions of 17 to 1,000 rows (every projection kernel),
    block tables that grow.  32-bit: the last rows against the plain implementation, and the cuttings
    bit for bit; bfloat16: the cuttings bit for bit.  Then eight requests decoding together from
    captured graphs while their block tables cross a captured width: the same bits as their whole prompts."""
    from vosti_amd.cache import CachePool
    from vosti_amd.engine import ModelRunner, StepEntry
    from vosti_amd.engine.step import width_bucket
    from vosti_amd.models import load_model
    d, V = full_width_dir, FULL_WIDTH["vocab_size"]
    rng = random.Random(77)
    long = [rng.randrange(V) for _ in range(2400)]
    pages = -(-2400 // 64)
    keep = list(range(2400 - 40, 2400)) + [0, 63, 64, 255, 256, 1023, 1024, 2047, 2048]      # rows compared
    for dtype_name in ("float32", "bfloat16"):
        runner = make_runner(d, dtype_name, 64, num_pages=pages)
        whole = replay(runner, [([(0, long, sorted(keep))], [0])])
        if dtype_name == "float32":
            ref = PlainQwen3(d, torch.float32).logits(long)
            got = torch.stack([whole[(0, j)] for j in range(2400 - 16, 2400)])
            torch.testing.assert_close(got, ref[2400 - 16:], **TOL["float32"])
            del ref
        # All but the last 32 tokens in one step, then token by token.
        steps = [([(0, long[:2368], [j for j in sorted(keep) if j < 2368])], [])]
        steps += [([(0, long[j:j + 1], [0])], [0] if j == 2399 else []) for j in range(2368, 2400)]
        tail = replay(runner, steps)
        # Portions of changing size.
        sizes, pos, steps = (700, 33, 64, 2, 129, 511, 40, 17, 1000, 5), 0, []
        k = 0
        while pos < 2400:
            n = min(sizes[k % len(sizes)], 2400 - pos)
            k += 1
            steps.append(([(0, long[pos:pos + n], [j - pos for j in sorted(keep) if pos <= j < pos + n])], [0] if pos + n == 2400 else []))
            pos += n
        chunks = replay(runner, steps)
        for label, got in (("tail", tail), ("chunks", chunks)):
            assert set(got) == set(whole), (dtype_name, label)
            bad = [key for key in sorted(whole) if not torch.equal(got[key], whole[key])]
            assert not bad, f"{dtype_name}, {label}: first differing (request, position) {bad[0]} of {len(bad)}"
        del runner, whole, tail, chunks

    # Eight requests decode together under graph replay while their tables grow from 16 to 17 pages,
    # which a capture of 16 pages does not hold: first an eager step, then a capture, then replays again.
    assert width_bucket(16) == 16 and width_bucket(17) == 24
    model = load_model(d, "bfloat16")
    seqs = [[rng.randrange(V) for _ in range(1040 + i)] for i in range(8)]
    heads = [len(sq) - 44 for sq in seqs]                    # 996 .. 1003 tokens before the decoded ones
    pool = CachePool(model, page_size=64, num_pages=8 * 17 + 1, num_slots=9)
    eager = ModelRunner(model, pool)
    want = {}
    for i, sq in enumerate(seqs):
        rows = list(range(heads[i], len(sq)))
        logits = eager.kernels.to_f32(eager.step([StepEntry(i, sq, rows)])).cpu()
        want.update({(i, j): logits[n] for n, j in enumerate(rows)})
        eager.finish(i)
    g = ModelRunner(model, pool, graphs=True)
    for i, sq in enumerate(seqs):
        g.step([StepEntry(100 + i, sq[:heads[i]], [])])
    for t in range(44):
        logits = g.kernels.to_f32(g.step([StepEntry(100 + i, [sq[heads[i] + t]], [0]) for i, sq in enumerate(seqs)])).cpu()
        for i in range(8):
            assert torch.equal(logits[i], want[(i, heads[i] + t)]), (t, i)
    st = g.graph_stats
    assert st["captured"] == 2 and st["replayed"] >= 38, st
    assert {key[1][0] for key in g._captured} == {16, 24}
    for i in range(8):
        g.finish(100 + i)
    assert pool.manager.num_requests() == 0 and pool.manager.check() == ""


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_trace_run_prefix_reuse_is_bit_identical_to_a_cold_run(tiny_dirs, tmp_path, name, dtype_name):
    """The fourth relation of the reference's determinism protocol, cold against warm
    (scripts/determinism_tests/protocol.py:26): request b after request a, which shares its first 70
    tokens; with reuse, b's shared full pages are not computed again, and every logit of b that is
    computed is the cold run's, bit for bit."""
    cfg, page, _ = TINY[name]
    vocab = cfg["vocab_size"]
    rng = random.Random(5 + ord(name))
    shared = [rng.randrange(vocab) for _ in range(70)]
    a = shared + [rng.randrange(vocab) for _ in range(9)]
    b = shared + [rng.randrange(vocab) for _ in range(21)]
    want_b = list(range(len(b)))

    def run(out, warm):
        steps = [{"step": 0, "entries": [{"id": "a", "prompt": a, "tokens": a, "want": [len(a) - 1]}], "end": ["a"]},
                 {"step": 1, "entries": [{"id": "b", "prompt": b, "tokens": b[:80], "want": [w for w in want_b if w < 80]}], "end": []},
                 {"step": 2, "entries": [{"id": "b", "tokens": b[80:], "want": [w - 80 for w in want_b if w >= 80]}], "end": ["b"]}]
        extra = (["--prefix-cache", "--prefix-report", str(out / "report.txt")] if warm else []) + ["--engine", which]
        run_trace(tiny_dirs[name], dtype_name, out, max_tokens=256, steps=steps, page_size=page, extra=extra)
        return [np.fromfile(out / f"{s}.f32", dtype="<f4").reshape(-1, vocab) for s in range(3)]

    for which in ("python", "native"):        # the two step functions, each cold against warm
        cold_dir, warm_dir = tmp_path / f"cold_{which}", tmp_path / f"warm_{which}"
        cold_dir.mkdir(); warm_dir.mkdir()
        cold, warm = run(cold_dir, False), run(warm_dir, True)
        report = dict(line.split() for line in (warm_dir / "report.txt").read_text().splitlines())
        cached = 70 // page * page
        assert report == {"a": "0", "b": str(cached)} and cached > 0          # b found a's pages
        assert np.array_equal(warm[0], cold[0])
        assert warm[1].shape[0] == 80 - cached and np.array_equal(warm[1], cold[1][cached:])    # the cached tokens are not run
        assert np.array_equal(warm[2], cold[2])


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_a_model_without_layers(tmp_path, dtype_name):
    """num_hidden_layers 0: logits = head(norm(embedding)) (src/exec/dense_swiglu_model.rs:276-359)."""
    from vosti_amd.config import Qwen3Config
    from vosti_amd.engine import Engine
    from vosti_amd.sampling import SamplingParams
    from vosti_amd.weights import write_random_model
    cfg = Qwen3Config(**dict(TINY["B"][0], num_hidden_layers=0))
    write_random_model(cfg, 6, tmp_path, dtype=torch.bfloat16)
    rng = random.Random(1)
    prompts = [[rng.randrange(cfg.vocab_size) for _ in range(n)] for n in (1, 30, 71)]
    runner = make_runner(tmp_path, dtype_name, 16, num_pages=8)
    assert runner.pool.entries == [] and runner.model.layers == []
    whole = replay(runner, cut_whole(prompts))
    plain, exact = PlainQwen3(tmp_path, DTYPES[dtype_name]), PlainQwen3(tmp_path, torch.float32)
    for i, p in enumerate(prompts):
        got = torch.stack([whole[(i, j)] for j in range(len(p))])
        assert_matches_plain(got, plain.logits(p), exact.logits(p), dtype_name, f"request {i}")
    got = replay(runner, cut_chunks(prompts))
    assert all(torch.equal(got[key], whole[key]) for key in whole)
    out = Engine(tmp_path, dtype=dtype_name, num_pages=8, page_size=16, max_num_seqs=2).generate(prompts[:2], SamplingParams(max_tokens=3))
    assert [len(o) for o in out] == [3, 3]


def test_decode_scratch_follows_the_decoded_rows_not_the_step(tiny_dirs):
    """A long prompt portion beside two decoded tokens: the attention's scratch is asked for the two
    tokens, not for every row of the step."""
    from vosti_amd.engine import StepEntry
    name = "C"
    prompts = prompts_for(name)
    runner = make_runner(tiny_dirs[name], "bfloat16", 64, num_pages=20)
    runner.step([StepEntry(1, prompts[3][:129], []), StepEntry(2, prompts[4][:200], [])])
    entries = [StepEntry(0, prompts[6][:400], [399]), StepEntry(1, prompts[3][129:130], [0]), StepEntry(2, prompts[4][200:201], [0])]
    runner.begin(entries)
    lay = runner._layout(entries)
    mixer = runner.model.layers[0].mixer
    two = runner.kernels.attn_scratch_floats(2, mixer.nq, mixer.d, 1)
    assert runner.workspace_needed(lay.host) == two < runner.kernels.attn_scratch_floats(402, mixer.nq, mixer.d, 1) // 100
    calls = []
    real = runner._get_workspace
    runner._get_workspace = lambda n: (calls.append(n), real(n))[1]
    runner.run(entries)
    runner.end(entries)
    assert calls and max(calls) == two
