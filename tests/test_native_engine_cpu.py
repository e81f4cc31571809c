"""The native engine's reading of config.json and of weight files, and the rules it shares with the Python
package, on the CPU.

``vosti_engine --kind describe`` prints what the program makes of a model folder without touching a GPU.  The
rules of an architecture are written once, in the native library, and the Python package asks the library for
them; the weight files are read by two readers (the safetensors package there, a reader of its own here), which
must agree."""
import json
import subprocess

import pytest

from conftest import TINY
from test_config_weights_cpu import hf_dict
from vosti_amd.config import ConfigError, Qwen3Config, config_from_dict
from vosti_amd.kernels import build
from vosti_amd.models.decoder import DecoderModel
from vosti_amd.weights import open_checkpoint


@pytest.fixture(scope="module")
def program():
    return str(build.ensure("engine", verbose=False))


def describe(program, folder):
    return subprocess.run([program, "--kind", "describe", "--model-path", str(folder)], capture_output=True, text=True)


class NoKernels:
    name, dtype = "none", None


@pytest.mark.parametrize("name", sorted(TINY))
def test_description_agrees_with_the_python_package(program, tiny_dirs, name):
    d = tiny_dirs[name]
    r = describe(program, d)
    assert r.returncode == 0, r.stderr
    got = json.loads(r.stdout)
    cfg = TINY[name][0]
    spec = Qwen3Config(**cfg).model_spec()
    # What the description must hold, written out here from the configuration's numbers.
    L = cfg["num_hidden_layers"]
    per_layer = ["input_layernorm.weight", "post_attention_layernorm.weight", "mlp.down_proj.weight", "mlp.gate_proj.weight",
                 "mlp.up_proj.weight", "self_attn.k_norm.weight", "self_attn.k_proj.weight", "self_attn.o_proj.weight",
                 "self_attn.q_norm.weight", "self_attn.q_proj.weight", "self_attn.v_proj.weight"]
    names = [f"model.layers.{i}.{n}" for i in range(L) for n in per_layer] + ["model.embed_tokens.weight", "model.norm.weight"]
    if not cfg["tie_word_embeddings"]:
        names.append("lm_head.weight")
    assert got["tensor_names"] == sorted(names)
    mixer = spec.layers[0].mixer.params
    assert (mixer["num_heads"], mixer["num_kv_heads"], mixer["head_dim"]) == (cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"])
    assert mixer["scale"] == cfg["head_dim"] ** -0.5 and mixer["window"] == 0
    assert mixer["q_norm"].params == mixer["k_norm"].params == {"size": cfg["head_dim"], "eps": cfg["rms_norm_eps"]}
    assert mixer["position"].params == {"head_dim": cfg["head_dim"], "rotary_dim": cfg["head_dim"], "theta": cfg["rope_theta"],
                                        "max_positions": cfg["max_position_embeddings"]}
    assert spec.layers[0].norms["input"].params == {"size": cfg["hidden_size"], "eps": cfg["rms_norm_eps"]} == spec.final_norm.params
    assert spec.layers[0].feed_forward.params == {"hidden_size": cfg["hidden_size"], "intermediate_size": cfg["intermediate_size"]}
    assert [(e.layer, e.cache_from) for e in spec.schedule] == [(i, None) for i in range(L)]
    assert got["architecture"] == spec.architecture == "Qwen3ForCausalLM"
    assert (got["vocab_size"], got["hidden_size"], got["max_positions"]) == (spec.vocab_size, spec.hidden_size, spec.max_positions)
    assert got["layers"] == len(spec.layers) and got["schedule"] == len(spec.schedule)
    expected = DecoderModel(spec, NoKernels()).expected_tensors()
    assert got["tensor_names"] == sorted(expected)
    assert got["ignored_names"] == list(spec.ignored_names)
    # The program's own safetensors reader sees the tensors the safetensors package sees.
    ck = open_checkpoint(d)
    assert {n: (e["dtype"], tuple(e["shape"])) for n, e in got["stored"].items()} == {n: (dt, shape) for n, (_, shape, dt) in ck.entries.items()}


BAD = [
    (dict(num_key_value_heads=3), "must be a multiple of 'num_key_value_heads'"),
    (dict(head_dim=15), "must be even"),
    (dict(hidden_act="gelu"), "this architecture uses 'silu'"),
    (dict(attention_bias=True), "'attention_bias' must be false"),
    (dict(use_sliding_window=True), "'use_sliding_window' must be false"),
    (dict(rope_scaling={"rope_type": "yarn", "factor": 4.0}), "'rope_scaling' must be null"),
    (dict(num_hidden_layers=-1), "'num_hidden_layers' must be an integer, zero or more"),
    (dict(vocab_size=0), "'vocab_size' must be a positive integer"),
    (dict(rms_norm_eps=0.0), "'rms_norm_eps' must be a finite positive number"),
    (dict(architectures=["LlamaForCausalLM"]), "unknown architecture 'LlamaForCausalLM'"),
    (dict(tie_word_embeddings="yes"), "'tie_word_embeddings' must be true or false"),
]


@pytest.mark.parametrize("over,message", BAD)
def test_both_readers_refuse_the_same_configurations(program, tmp_path, over, message):
    raw = hf_dict(TINY["A"][0], **over)
    (tmp_path / "config.json").write_text(json.dumps(raw))
    r = describe(program, tmp_path)
    assert r.returncode == 1 and message in r.stderr, r.stderr
    with pytest.raises(ConfigError) as e:
        config_from_dict(raw)
    assert message in str(e.value)


def test_missing_keys_defaults_and_zero_layers(program, tmp_path):
    raw = hf_dict(TINY["B"][0])
    del raw["rope_theta"]
    (tmp_path / "config.json").write_text(json.dumps(raw))
    r = describe(program, tmp_path)
    assert r.returncode == 1 and "required key 'rope_theta' is missing" in r.stderr
    # Newer spelling of theta, no head_dim, no kv head count, no layers, the architecture by model_type alone.
    raw = hf_dict(TINY["A"][0], rope_parameters={"rope_theta": 1e4, "rope_type": "default"}, num_hidden_layers=0)
    for key in ("rope_theta", "head_dim", "num_key_value_heads", "architectures"):
        del raw[key]
    (tmp_path / "config.json").write_text(json.dumps(raw))
    r = describe(program, tmp_path)
    assert r.returncode == 0, r.stderr
    got = json.loads(r.stdout)
    assert got["layers"] == 0 and got["tensor_names"] == ["model.embed_tokens.weight", "model.norm.weight"]
    (tmp_path / "config.json").write_text("{not json")
    assert describe(program, tmp_path).returncode == 1


def test_random_streams_have_the_python_package_seeds(program, tiny_dirs):
    """The seed of a tensor's random stream is a BLAKE2b digest of "<seed>:<name>"; the program computes it
    with code of its own."""
    from vosti_amd.weights.random_init import tensor_seed
    r = subprocess.run([program, "--kind", "describe", "--model-path", str(tiny_dirs["B"]), "--random-weights", "20250101"],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    got = json.loads(r.stdout)
    assert [int(t) for t in got["tensor_seeds"]] == [tensor_seed(20250101, n) for n in got["tensor_names"]]


def test_usage_errors(program, tmp_path):
    r = subprocess.run([program, "--family", "qwen3"], capture_output=True, text=True, env={})
    assert r.returncode == 2 and "MODEL_PATH (or --model-path) is required" in r.stderr
    r = subprocess.run([program, "--family", "llama", "--model-path", str(tmp_path)], capture_output=True, text=True, env={})
    assert r.returncode == 2 and "unknown --family llama (one of: qwen3)" in r.stderr
    r = subprocess.run([program, "--family", "qwen3", "--model-path", str(tmp_path), "--colour", "blue"], capture_output=True, text=True, env={})
    assert r.returncode == 2 and "unknown option --colour" in r.stderr


def _write_safetensors(path, header: dict, data: bytes = b"\0" * 64):
    text = json.dumps(header).encode()
    path.write_bytes(len(text).to_bytes(8, "little") + text + data)


MALFORMED = [
    ({"w": {"dtype": "F32", "shape": [4], "data_offsets": [-16, 0]}}, "data offsets that are no sizes"),
    ({"w": {"dtype": "F32", "shape": [4], "data_offsets": [0, 1 << 40]}}, "lies outside the file"),
    ({"w": {"dtype": "F32", "shape": [-4], "data_offsets": [0, 16]}}, "a shape entry that is no size"),
    ({"w": {"dtype": "F32", "shape": [1 << 40, 1 << 40], "data_offsets": [0, 16]}}, "larger than any file"),
    ({"w": {"dtype": "F32", "shape": [1 << 62, 4], "data_offsets": [0, 16]}}, "larger than any file"),
    ({"w": {"dtype": "F32", "shape": [5], "data_offsets": [0, 16]}}, "its shape needs 20"),
    ({"w": {"dtype": "F32", "shape": [4], "data_offsets": [32, 16]}}, "lies outside the file"),
]


@pytest.mark.parametrize("header,message", MALFORMED)
def test_a_malformed_safetensors_header_is_refused(program, tmp_path, header, message):
    """Offsets and sizes in a file's header are checked before they become addresses: negative ones, ones
    beyond the file and shapes whose product overflows are errors, not reads outside the mapping."""
    (tmp_path / "config.json").write_text(json.dumps(hf_dict(TINY["A"][0])))
    _write_safetensors(tmp_path / "model.safetensors", header)
    r = describe(program, tmp_path)
    assert r.returncode == 1 and message in r.stderr, r.stderr


def test_rotation_frequencies_are_the_reference_formula():
    """inv_freq = 1 / theta^(arange(0, D, 2) / D) in 32-bit (python/vosti_kernels/rotary.py:80-90).  The library's
    routine, which both step functions use, gives the 32-bit number nearest to the exact power (so it does not
    depend on whose pow runs): equal to the formula evaluated in 64-bit and rounded, and within one step of
    the type of what torch's 32-bit pow gives."""
    import numpy as np
    import torch
    from vosti_amd.cache.host import rotary_inverse_frequencies
    for theta, dim in ((1e4, 16), (1e6, 32), (5e5, 64), (1e6, 128), (1e4, 256), (123456.789, 80)):
        got = rotary_inverse_frequencies(theta, dim)
        exponent = (np.arange(0, dim, 2, dtype=np.float32) / np.float32(dim)).astype(np.float32)
        power = np.power(np.float64(np.float32(theta)), exponent.astype(np.float64)).astype(np.float32)
        assert np.array_equal(got, (np.float32(1.0) / power).astype(np.float32)), (theta, dim)
        formula = (1.0 / (float(theta) ** (torch.arange(0, dim, 2, dtype=torch.int64).to(torch.float32) / dim))).numpy()
        steps = np.abs(got.view(np.int32).astype(np.int64) - formula.view(np.int32).astype(np.int64))
        assert got[0] == 1.0 and steps.max() <= 1, (theta, dim, steps.max())


def test_recording_sizes_are_the_library_s():
    from vosti_amd.cache.host import graph_row_bucket, graph_width_bucket, max_graphs
    assert [graph_row_bucket(n) for n in (1, 2, 3, 4, 5, 6, 7, 8, 9, 12, 13, 16, 17, 24, 25, 33, 48, 49, 64, 65, 512, 513, 700)] == \
        [1, 2, 3, 4, 6, 6, 8, 8, 12, 12, 16, 16, 24, 24, 32, 48, 48, 64, 64, 96, 512, 513, 700]
    assert [graph_width_bucket(p) for p in (0, 1, 8, 9, 16, 17, 24, 25, 33, 48, 49)] == [8, 8, 8, 16, 16, 24, 24, 32, 48, 48, 64]
    assert max_graphs() == 24


def test_an_architecture_of_the_library_needs_no_python_class(tmp_path):
    """A config.json whose architecture the Python package has no class for is read through the native library
    (here: Qwen3 with the Python class taken out of the registry)."""
    from vosti_amd.config import registry
    raw = hf_dict(TINY["B"][0])
    saved = registry._ARCHITECTURES.pop("Qwen3ForCausalLM")
    try:
        cfg = config_from_dict(raw)
        assert type(cfg).__name__ == "NativeConfig" and cfg.head_dim == 32 and cfg.rms_norm_eps == 1e-5
        assert cfg.model_spec() == saved.from_dict(raw).model_spec()
        assert registry.model_types()["qwen3"] == "Qwen3ForCausalLM"
        with pytest.raises(ConfigError, match="unknown architecture 'LlamaForCausalLM'"):
            config_from_dict(dict(raw, architectures=["LlamaForCausalLM"]))
    finally:
        registry._ARCHITECTURES["Qwen3ForCausalLM"] = saved
