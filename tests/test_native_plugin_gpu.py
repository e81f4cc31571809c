"""A position encoding and an architecture that the native engine's files know nothing of, brought in a plugin
(tests/toy_plugin.cpp): registered, built and stepped without a change to the engine's files.  The attention part
cannot run this encoding inside its fused launch (it offers no tables), so it runs head norms, encoding and cache
store step by step, each sub-part through its own methods."""
import json
import shutil

import pytest
import torch

import plain_qwen3 as plain
from conftest import ROOT, TINY
from test_model_gpu import DTYPES, assert_matches_plain, cut_chunks, cut_mixed, cut_tail, cut_whole, prompts_for, replay

pytestmark = pytest.mark.gpu

FACTOR = 4.0


@pytest.fixture(scope="module")
def plugin(tmp_path_factory):
    from vosti_amd.kernels import build
    return build.build_plugin(ROOT / "tests" / "toy_plugin.cpp", tmp_path_factory.mktemp("plugin") / "toy_plugin.so")


@pytest.fixture(scope="module")
def toy_dirs(tiny_dirs, tmp_path_factory):
    """The tiny Qwen3 folders with the toy architecture's name in config.json (the tensors are the same)."""
    out = {}
    for name in ("B", "C"):
        d = tmp_path_factory.mktemp(f"toy_{name}")
        shutil.copy(tiny_dirs[name] / "model.safetensors", d / "model.safetensors")
        raw = json.loads((tiny_dirs[name] / "config.json").read_text())
        raw.update(architectures=["ToyScaledRopeForCausalLM"], model_type="toy_scaled_rope", toy_rope_factor=FACTOR)
        (d / "config.json").write_text(json.dumps(raw))
        out[name] = d
    return out


class PlainToy(plain.PlainQwen3):
    """The plain decoder with the toy encoding: the first half of each head rotated, at positions / FACTOR."""

    def __init__(self, model_dir, dtype):
        super().__init__(model_dir, dtype)
        rot = self.d // 2
        inv_freq = 1.0 / (float(self.theta) ** (torch.arange(0, rot, 2, dtype=torch.int64).to(torch.float32) / rot))
        pos = torch.arange(self.cfg["max_position_embeddings"], dtype=torch.int64).to(torch.float32) / FACTOR
        ang = pos[:, None] * inv_freq[None, :]
        self.cos, self.sin = ang.cos().to(dtype).float(), ang.sin().to(dtype).float()


def test_the_toy_encoding_is_another_model(toy_dirs, tiny_dirs):
    ids = prompts_for("B")[3]
    assert (PlainToy(toy_dirs["B"], torch.float32).logits(ids) - plain.PlainQwen3(tiny_dirs["B"], torch.float32).logits(ids)).abs().max() > 1e-3


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "C"])
def test_a_plugin_s_position_encoding_through_the_native_step_function(plugin, toy_dirs, name, dtype_name):
    from test_native_engine_gpu import _NativeRunner
    from vosti_amd.engine import create_engine
    from vosti_amd.engine.native import NativeEngine, load_plugin, native_support
    from vosti_amd.sampling import SamplingParams
    d, page = toy_dirs[name], TINY[name][1]
    load_plugin(plugin)
    assert native_support(d) == (True, "")
    prompts = prompts_for(name)
    toy, exact = PlainToy(d, DTYPES[dtype_name]), PlainToy(d, torch.float32)
    runner = _NativeRunner(d, dtype_name, page, -(-max(map(len, prompts)) // page))
    whole = replay(runner, cut_whole(prompts))
    for i, p in enumerate(prompts):
        got = torch.stack([whole[(i, j)] for j in range(len(p))])
        assert_matches_plain(got, toy.logits(p), exact.logits(p), dtype_name, f"request {i} (length {len(p)}), whole, toy encoding")
    mixed_steps, mixed_pages = cut_mixed(prompts, page)
    for label, steps, n in (("tail", cut_tail(prompts), None), ("chunks", cut_chunks(prompts), None), ("mixed", mixed_steps, mixed_pages)):
        if n is not None:
            runner = _NativeRunner(d, dtype_name, page, n)
        got = replay(runner, steps)
        bad = [k for k in sorted(whole) if not torch.equal(got[k], whole[k])]
        assert set(got) == set(whole) and not bad, f"{label}: first differing (request, position) {bad[:1]} of {len(bad)}"
    # Generation through the entry point, which finds the native engine able to run it, with recorded decode steps.
    e = create_engine(d, dtype=dtype_name, num_pages=64, page_size=page, max_num_seqs=3, graphs=True)
    assert isinstance(e, NativeEngine)
    ps = [prompts[1], prompts[3][:40], prompts[2]]
    outs = e.generate(ps, SamplingParams(max_tokens=12, ignore_eos=True))
    assert e.stats()["graph_stats"]["replayed"] > 0
    if dtype_name == "float32":
        assert outs == [exact.generate_greedy(p, 12) for p in ps]


def test_without_the_plugin_the_architecture_is_unknown(toy_dirs, tmp_path):
    """A process that has not loaded the plugin (the engine's program, started without --plugin) refuses the folder
    and names what is registered; with --plugin it generates."""
    import subprocess
    from vosti_amd.kernels import build
    program = str(build.ensure("engine", verbose=False))
    lib = build.ensure("f32", verbose=False)
    args = [program, "--family", "toy_scaled_rope", "--dtype", "float32", "--lib-dir", str(lib.parent), "--model-path", str(toy_dirs["B"]),
            "--prompt-ids", "5,17,3,99", "--max-tokens", "6", "--page-size", "8"]
    r = subprocess.run(args, capture_output=True, text=True, timeout=110, env={})
    assert r.returncode == 2 and "unknown --family toy_scaled_rope (one of: qwen3)" in r.stderr
    so = build.build_plugin(ROOT / "tests" / "toy_plugin.cpp", tmp_path / "toy_plugin.so")
    r = subprocess.run(args + ["--plugin", str(so)], capture_output=True, text=True, timeout=110, env={})
    assert r.returncode == 0, r.stderr[-2000:]
    out = json.loads([l for l in r.stdout.splitlines() if l.startswith("MODEL_OUTPUT_TOKEN_IDS=")][0].split("=", 1)[1])
    assert out == PlainToy(toy_dirs["B"], torch.float32).generate_greedy([5, 17, 3, 99], 6)


# ----------------------------------------------------------------- a hybrid toy architecture, natively
HYBRID = dict(architectures=["ToyNativeHybridForCausalLM"], model_type="toy_native_hybrid", vocab_size=211, hidden_size=80, heads=4,
              kv_heads=2, head_dim=32, inter=112, max_positions=256, eps=1e-5, theta=1e4, window=20, rope_factor=2.0, scale=0.2)
HYBRID_SCHEDULE = [(0, None), (1, None), (2, None), (0, None), (2, 2)]       # (layer, the entry whose keys and values it reads)


def write_hybrid(out):
    """config.json and model.safetensors of the hybrid toy, written here: the tensor names are the plugin's."""
    from safetensors.torch import save_file
    c = HYBRID
    H, d, nq, nkv, I, V = c["hidden_size"], c["head_dim"], c["heads"], c["kv_heads"], c["inter"], c["vocab_size"]
    g = torch.Generator().manual_seed(11)
    # Values that bfloat16 holds exactly, stored in 32-bit: whichever tensors a loader keeps in 32-bit, the model is the same.
    normal = lambda *shape, std=0.08: (torch.randn(*shape, generator=g) * std).to(torch.bfloat16).float()
    gain = lambda n: (0.5 + torch.rand(n, generator=g)).to(torch.bfloat16).float()
    t = {"emb": normal(V, H, std=0.5), "norm": gain(H), "head": normal(V, H)}
    for i in range(3):
        t[f"l{i}.n1"], t[f"l{i}.n2"] = gain(H), gain(H)
        t[f"l{i}.ffn.gate_proj.weight"], t[f"l{i}.ffn.up_proj.weight"] = normal(I, H), normal(I, H)
        t[f"l{i}.ffn.down_proj.weight"] = normal(H, I)
        if i == 1:
            t["l1.mixer.in_proj.weight"], t["l1.mixer.gain"] = normal(H, H), gain(H)
            continue
        t[f"l{i}.mixer.q_proj.weight"], t[f"l{i}.mixer.o_proj.weight"] = normal(nq * d, H, std=0.2), normal(H, nq * d)
        t[f"l{i}.mixer.k_proj.weight"], t[f"l{i}.mixer.v_proj.weight"] = normal(nkv * d, H, std=0.2), normal(nkv * d, H)
        if i == 0:
            t["l0.mixer.q_norm.weight"], t["l0.mixer.k_norm.weight"] = gain(d), gain(d)
    (out / "config.json").write_text(json.dumps(c))
    save_file({n: x.contiguous() for n, x in t.items()}, str(out / "model.safetensors"))
    return out


@pytest.fixture(scope="module")
def hybrid_dir(tmp_path_factory):
    return write_hybrid(tmp_path_factory.mktemp("hybrid"))


class PlainHybrid:
    """The hybrid toy on whole sequences, from the plain parts: what tests/toy_plugin.cpp says it computes."""

    def __init__(self, model_dir, dtype):
        from safetensors.torch import load_file
        self.c, self.dtype = json.loads((model_dir / "config.json").read_text()), dtype
        self.w = {n: x.float().to(dtype).float() for n, x in load_file(str(model_dir / "model.safetensors")).items()}
        c = self.c
        self.rope = plain.rope_tables(c["max_positions"], c["head_dim"], c["theta"], dtype)
        rot = c["head_dim"] // 2
        inv_freq = 1.0 / (float(c["theta"]) ** (torch.arange(0, rot, 2, dtype=torch.int64).to(torch.float32) / rot))
        ang = (torch.arange(c["max_positions"], dtype=torch.int64).to(torch.float32)[:, None] * (inv_freq / c["rope_factor"])[None, :])
        self.toy_rope = ang.cos().to(dtype).float(), ang.sin().to(dtype).float()

    def attention_layer(self, i, x, positions, kv):
        c, w, dt = self.c, self.w, self.dtype
        T, nq, nkv, d = x.shape[0], c["heads"], c["kv_heads"], c["head_dim"]
        p = f"l{i}.mixer."
        q = plain.linear(x, w[p + "q_proj.weight"], dt).view(T, nq, d)
        k = plain.linear(x, w[p + "k_proj.weight"], dt).view(T, nkv, d)
        v = plain.linear(x, w[p + "v_proj.weight"], dt).view(T, nkv, d)
        if i == 0:
            q, k = plain.head_rms_norm(q, w[p + "q_norm.weight"], c["eps"], dt), plain.head_rms_norm(k, w[p + "k_norm.weight"], c["eps"], dt)
        cos, sin = self.rope if i == 0 else self.toy_rope
        q, k = plain.apply_rope(q, cos, sin, positions, dt), plain.apply_rope(k, cos, sin, positions, dt)
        if kv is not None:
            k, v = kv
        out = plain.attention(q, k, v, c["scale"], dt, window=0 if i == 0 else c["window"])
        return plain.linear(out.reshape(T, nq * d), w[p + "o_proj.weight"], dt), (k, v)

    def carry_layer(self, x):
        z = plain.linear(x, self.w["l1.mixer.in_proj.weight"], self.dtype)
        state, ys = torch.zeros(1, x.shape[1]), []
        for t in range(x.shape[0]):
            y, state = plain.add_rms_norm(z[t:t + 1], state, self.w["l1.mixer.gain"], self.c["eps"], self.dtype)
            ys.append(y)
        return torch.cat(ys)

    def logits(self, ids):
        c, w, dt = self.c, self.w, self.dtype
        positions = torch.arange(len(ids))
        hidden, residual, stored = plain.embedding(torch.tensor(ids), w["emb"]), None, {}
        for entry, (i, reads) in enumerate(HYBRID_SCHEDULE):
            if residual is None:
                residual, normed = hidden, plain.rms_norm(hidden, w[f"l{i}.n1"], c["eps"], dt)
            else:
                normed, residual = plain.add_rms_norm(hidden, residual, w[f"l{i}.n1"], c["eps"], dt)
            if i == 1:
                mixed = self.carry_layer(normed)
            else:
                mixed, stored[entry] = self.attention_layer(i, normed, positions, stored[reads] if reads is not None else None)
            normed, residual = plain.add_rms_norm(mixed, residual, w[f"l{i}.n2"], c["eps"], dt)
            gu = torch.cat([plain.linear(normed, w[f"l{i}.ffn.gate_proj.weight"], dt), plain.linear(normed, w[f"l{i}.ffn.up_proj.weight"], dt)], 1)
            hidden = plain.linear(plain.swiglu(gu, dt), w[f"l{i}.ffn.down_proj.weight"], dt)
        final, _ = plain.add_rms_norm(hidden, residual, w["norm"], c["eps"], dt)
        return plain.linear(final, w["head"], dt)

    def generate_greedy(self, prompt, n_new):
        ids = list(prompt)
        for _ in range(n_new):
            ids.append(plain.argmax_token(self.logits(ids)[-1]))
        return ids[len(prompt):]


def hybrid_prompts():
    import random
    rng = random.Random(5)
    return [[rng.randrange(HYBRID["vocab_size"]) for _ in range(n)] for n in (3, 29, 64, 150, 41)]


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_a_hybrid_toy_through_the_native_step_function(plugin, hybrid_dir, dtype_name):
    """A mixer with state of its own in a state slot, a windowed attention layer beside an all-keys one (two groups
    of pages), a layer that runs twice and an execution that reads another's keys and values, all from a plugin:
    the whole prompts match a plain implementation written here, and every other cutting gives the same bits."""
    from test_native_engine_gpu import _NativeRunner
    from vosti_amd.engine import create_engine
    from vosti_amd.engine.native import NativeEngine, load_plugin, native_support
    from vosti_amd.sampling import SamplingParams
    load_plugin(plugin)
    assert native_support(hybrid_dir) == (True, "")
    page, prompts = 8, hybrid_prompts()
    toy, exact = PlainHybrid(hybrid_dir, DTYPES[dtype_name]), PlainHybrid(hybrid_dir, torch.float32)
    runner = _NativeRunner(hybrid_dir, dtype_name, page, -(-max(map(len, prompts)) // page))
    whole = replay(runner, cut_whole(prompts))
    for i, p in enumerate(prompts):
        got = torch.stack([whole[(i, j)] for j in range(len(p))])
        assert_matches_plain(got, toy.logits(p), exact.logits(p), dtype_name, f"request {i} (length {len(p)}), whole, hybrid toy")
    mixed_steps, mixed_pages = cut_mixed(prompts, page)
    for label, steps, n in (("tail", cut_tail(prompts), None), ("chunks", cut_chunks(prompts), None), ("mixed", mixed_steps, mixed_pages)):
        if n is not None:
            runner = _NativeRunner(hybrid_dir, dtype_name, page, n)
        got = replay(runner, steps)
        bad = [k for k in sorted(whole) if not torch.equal(got[k], whole[k])]
        assert set(got) == set(whole) and not bad, f"{label}: first differing (request, position) {bad[:1]} of {len(bad)}"
        assert runner.engine.cache_check() == ""
    # Generation through the entry point: asked to record its decode steps, the engine does not, since the
    # state mixer says that it cannot be replayed.
    e = create_engine(hybrid_dir, dtype=dtype_name, num_pages=64, page_size=page, max_num_seqs=3, graphs=True)
    assert isinstance(e, NativeEngine)
    ps = [prompts[1], prompts[3][:40], prompts[2]]
    outs = e.generate(ps, SamplingParams(max_tokens=12, ignore_eos=True))
    assert e.stats()["graph_stats"]["captured"] == 0 and e.stats()["graph_stats"]["replayed"] == 0
    if dtype_name == "float32":
        assert outs == [exact.generate_greedy(p, 12) for p in ps]


def test_the_hybrid_s_state_and_window_matter(hybrid_dir):
    """The plain hybrid itself: without the carried state, or with all keys in the windowed layer, the logits differ,
    so that an engine that dropped either would fail the comparison above."""
    ids = hybrid_prompts()[2]
    ref = PlainHybrid(hybrid_dir, torch.float32)
    base = ref.logits(ids)

    class NoState(PlainHybrid):
        def carry_layer(self, x):
            z = plain.linear(x, self.w["l1.mixer.in_proj.weight"], self.dtype)
            return plain.rms_norm(z, self.w["l1.mixer.gain"], self.c["eps"], self.dtype)

    assert (NoState(hybrid_dir, torch.float32).logits(ids) - base).abs().max() > 1e-2
    wide = PlainHybrid(hybrid_dir, torch.float32)
    wide.c = dict(wide.c, window=0)
    assert (wide.logits(ids) - base)[HYBRID["window"] + 5:].abs().max() > 1e-3
    assert torch.equal(wide.logits(ids)[:HYBRID["window"]], base[:HYBRID["window"]])
