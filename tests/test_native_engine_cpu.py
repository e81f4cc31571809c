"""The native engine's reading of config.json and of weight files, on the CPU.

``vosti_engine --kind describe`` prints what the program makes of a model folder without touching a GPU;
it must agree with the Python package, which reads the same folder with other code (json and the
safetensors package there, a reader of its own here)."""
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
    spec = Qwen3Config(**TINY[name][0]).model_spec()
    assert got["architecture"] == spec.architecture
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
