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
