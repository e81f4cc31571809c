"""Configuration, registry and weight loading errors, on the CPU."""
import json

import pytest
import torch
from safetensors.torch import load_file, save_file

from conftest import TINY_A, TINY_B
from vosti_amd.config import ConfigError, Qwen3Config, architecture_names, config_from_dict, load_config
from vosti_amd.models.decoder import DecoderModel
from vosti_amd.weights import WeightError, open_checkpoint, write_random_model
from vosti_amd.weights.loader import check_against, convert
from vosti_amd.weights.random_init import expected_tensor_specs, random_tensor_cpu


def hf_dict(cfg, **over):
    d = dict(cfg, architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_act="silu", attention_bias=False,
             attention_dropout=0.0, use_sliding_window=False, sliding_window=None, rope_scaling=None)
    d.update(over)
    return d


def test_registry_and_round_trip():
    assert "Qwen3ForCausalLM" in architecture_names()
    c = config_from_dict(hf_dict(TINY_B))
    assert isinstance(c, Qwen3Config) and c.head_dim == 32 and c.rms_norm_eps == 1e-5 and not c.tie_word_embeddings
    assert config_from_dict(c.to_dict()) == c
    # model_type alone also names the architecture.
    d = hf_dict(TINY_A)
    del d["architectures"]
    assert config_from_dict(d).vocab_size == 256
    with pytest.raises(ConfigError, match="unknown architecture 'LlamaForCausalLM'"):
        config_from_dict(hf_dict(TINY_A, architectures=["LlamaForCausalLM"]))
    with pytest.raises(ConfigError, match="names no architecture"):
        config_from_dict({"hidden_size": 4})


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                                 "num_attention_heads", "max_position_embeddings", "rms_norm_eps", "rope_theta"])
def test_missing_key_is_named(key):
    d = hf_dict(TINY_A)
    del d[key]
    with pytest.raises(ConfigError, match=key):
        config_from_dict(d)


@pytest.mark.parametrize("over,match", [
    (dict(num_key_value_heads=3), "multiple"), (dict(head_dim=15), "even"), (dict(hidden_act="gelu"), "hidden_act"),
    (dict(attention_bias=True), "attention_bias"), (dict(use_sliding_window=True), "use_sliding_window"),
    (dict(rope_scaling={"rope_type": "yarn", "factor": 2.0}), "rope_scaling"), (dict(vocab_size=-1), "vocab_size"),
    (dict(rms_norm_eps=0), "rms_norm_eps"), (dict(tie_word_embeddings="yes"), "tie_word_embeddings"),
    (dict(model_type="llama"), "model_type"), (dict(num_hidden_layers=True), "num_hidden_layers"),
])
def test_bad_values_are_refused(over, match):
    # The reference's rules: python/vosti_kernels/model_families/qwen3/profile.py:129-164.
    with pytest.raises(ConfigError, match=match):
        config_from_dict(hf_dict(TINY_A, **over))


def test_defaults_and_newer_key_spellings():
    d = hf_dict(TINY_A)
    del d["head_dim"], d["rope_theta"], d["tie_word_embeddings"]
    d["rope_parameters"] = {"rope_type": "default", "rope_theta": 5000.0}
    c = config_from_dict(d)
    assert c.head_dim == 16 and c.rope_theta == 5000.0 and c.tie_word_embeddings is False


def test_model_spec_is_data():
    spec = Qwen3Config(**TINY_B).model_spec()
    assert len(spec.layers) == 3 and [e.layer for e in spec.schedule] == [0, 1, 2]
    m = spec.layers[1].mixer
    assert m.kind == "attention" and m.params["num_kv_heads"] == 2 and m.params["q_norm"].params["eps"] == 1e-5
    assert spec.layers[2].names["mixer.q_norm.weight"] == "model.layers.2.self_attn.q_norm.weight"
    assert not spec.head.params["tied"]


def test_load_config_errors(tmp_path):
    with pytest.raises(ConfigError, match="not found"):
        load_config(tmp_path)
    (tmp_path / "config.json").write_text("{")
    with pytest.raises(ConfigError, match="JSON"):
        load_config(tmp_path)


def test_random_weights_are_a_function_of_seed_and_name(tmp_path):
    a = write_random_model(Qwen3Config(**TINY_A), 0, tmp_path / "a")
    b = write_random_model(Qwen3Config(**TINY_A), 0, tmp_path / "b")
    c = write_random_model(Qwen3Config(**TINY_A), 1, tmp_path / "c")
    ta, tb, tc = (load_file(str(p / "model.safetensors")) for p in (a, b, c))
    assert set(ta) == set(expected_tensor_specs(Qwen3Config(**TINY_A)))
    assert "lm_head.weight" not in ta                                   # tied
    assert all(torch.equal(ta[n], tb[n]) for n in ta) and not torch.equal(ta["model.norm.weight"], tc["model.norm.weight"])
    assert ta["model.embed_tokens.weight"].dtype == torch.bfloat16
    w = ta["model.layers.0.mlp.down_proj.weight"].float()
    assert abs(w.std().item() - 0.02) < 2e-3 and abs(w.mean().item()) < 2e-3
    n = ta["model.norm.weight"].float()
    assert 0.9 - 2 ** -8 <= n.min() and n.max() <= 1.1 + 2 ** -7      # [0.9, 1.1), rounded to bfloat16
    # Any piece of a tensor can be drawn alone: the generator is counter-based.
    full = random_tensor_cpu(3, "x", (5000,), ("normal", 0.02))
    assert torch.equal(full, random_tensor_cpu(3, "x", (5000,), ("normal", 0.02)))
    assert json.loads((a / "config.json").read_text())["architectures"] == ["Qwen3ForCausalLM"]
    assert load_config(a) == Qwen3Config(**TINY_A)


def test_one_error_lists_missing_unexpected_and_misshapen(tmp_path):
    cfg = Qwen3Config(**TINY_B)
    d = write_random_model(cfg, 0, tmp_path / "m")
    t = load_file(str(d / "model.safetensors"))
    del t["model.layers.1.self_attn.k_norm.weight"], t["lm_head.weight"]
    t["model.layers.0.mlp.gate_proj.weight"] = t["model.layers.0.mlp.gate_proj.weight"][:, :-1].contiguous()
    t["model.layers.9.extra.weight"] = torch.zeros(2)
    save_file(t, str(d / "model.safetensors"))
    model = DecoderModel(cfg.model_spec(), None)
    with pytest.raises(WeightError) as e:
        check_against(model, open_checkpoint(d))
    msg = str(e.value)
    assert "missing (2): lm_head.weight, model.layers.1.self_attn.k_norm.weight" in msg
    assert "unexpected (1): model.layers.9.extra.weight" in msg
    assert "model.layers.0.mlp.gate_proj.weight: file has [224, 95], model needs [224, 96]" in msg


def test_sharded_folder_and_tied_head(tmp_path):
    cfg = Qwen3Config(**TINY_A)
    d = write_random_model(cfg, 0, tmp_path / "m")
    t = load_file(str(d / "model.safetensors"))
    names = sorted(t)
    save_file({n: t[n] for n in names[:10]}, str(d / "part1.safetensors"))
    save_file({n: t[n] for n in names[10:]} | {"lm_head.weight": t["model.embed_tokens.weight"]}, str(d / "part2.safetensors"))
    (d / "model.safetensors").unlink()
    index = {"weight_map": {n: ("part1.safetensors" if i < 10 else "part2.safetensors") for i, n in enumerate(names)}}
    (d / "model.safetensors.index.json").write_text(json.dumps(index))
    ckpt = open_checkpoint(d)
    check_against(DecoderModel(cfg.model_spec(), None), ckpt)          # a stored head beside a tied one is tolerated
    assert torch.equal(ckpt.read(["model.norm.weight"])["model.norm.weight"], t["model.norm.weight"])
    (d / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"a": "../outside.safetensors"}}))
    with pytest.raises(WeightError, match="outside"):
        open_checkpoint(d)
    with pytest.raises(WeightError, match="neither"):
        open_checkpoint(tmp_path)


def test_type_policy():
    f32, bf = torch.ones(3, dtype=torch.float32), torch.ones(3, dtype=torch.bfloat16)
    assert convert(f32, torch.bfloat16, keep_f32=False).dtype == torch.bfloat16
    assert convert(f32, torch.bfloat16, keep_f32=True).dtype == torch.float32      # stored in 32-bit: stays so
    assert convert(bf, torch.bfloat16, keep_f32=True).dtype == torch.bfloat16
    assert convert(bf, torch.float32, keep_f32=False).dtype == torch.float32
    assert convert(torch.ones(3, dtype=torch.int64), torch.bfloat16, keep_f32=False).dtype == torch.int32


def test_a_tied_head_is_the_embedding_by_name():
    """Tying lives in the specification: both parameters carry one tensor name, so they get one tensor."""
    tied, untied = Qwen3Config(**TINY_A).model_spec(), Qwen3Config(**TINY_B).model_spec()
    assert tied.names["head.weight"] == tied.names["embedding.weight"] == "model.embed_tokens.weight"
    assert tied.ignored_names == ("lm_head.weight",) and untied.ignored_names == ()
    assert untied.names["head.weight"] == "lm_head.weight"
    model = DecoderModel(tied, None)
    e = model.expected_tensors()["model.embed_tokens.weight"]
    assert [type(owner).__name__ for owner, _ in e.owners] == ["TokenEmbedding", "LinearHead"]
    t = {n: torch.zeros(x.spec.shape) for n, x in model.expected_tensors().items()}
    model.load_tensors(t)
    assert model.head.weight is model.embedding.weight
    # Sharers must agree on the shape.
    from dataclasses import replace
    from vosti_amd.config import PartSpec
    bad = replace(tied, head=PartSpec("linear_head", {"vocab_size": 255, "hidden_size": 64}))
    with pytest.raises(ValueError, match="shared by parameters of different shapes"):
        DecoderModel(bad, None).expected_tensors()


def test_zero_layers_is_a_configuration():
    # src/exec/dense_swiglu_model.rs:276-359; fixture tests/support/model_families/qwen3.rs:26-36.
    c = config_from_dict(hf_dict(TINY_A, num_hidden_layers=0))
    spec = c.model_spec()
    assert c.num_hidden_layers == 0 and spec.layers == () and spec.schedule == ()
    assert sorted(expected_tensor_specs(c)) == ["model.embed_tokens.weight", "model.norm.weight"]
    with pytest.raises(ConfigError, match="num_hidden_layers"):
        config_from_dict(hf_dict(TINY_A, num_hidden_layers=-1))


def test_launcher_families_come_from_the_registry():
    from vosti_amd.config import register_architecture
    from vosti_amd.launch import families
    assert families()["qwen3"] == "Qwen3ForCausalLM"

    @register_architecture("ProbeForCausalLM", model_type="probe_family")
    class Probe:
        pass
    assert families()["probe_family"] == "ProbeForCausalLM"


def test_multi_call_prompts_are_built_from_earlier_outputs():
    # The reference's own vector: examples/support/engine_calls.rs:130-141.
    from vosti_amd.launch import resolve_call_prompts
    call = {"label": "reuse", "max_tokens": 2, "output_prefix_from": {"call": 0, "request": 0, "count": 2, "suffix": [8]}}
    assert resolve_call_prompts(call, [([[1, 2]], [[3, 4, 5]])]) == [[1, 2, 3, 4, 8]]
    with pytest.raises(SystemExit):
        resolve_call_prompts(call, [])
    with pytest.raises(SystemExit):
        resolve_call_prompts(call, [([[1, 2]], [[3]])])
    assert resolve_call_prompts({"prompts": [[1, 2], [3]]}, []) == [[1, 2], [3]]
