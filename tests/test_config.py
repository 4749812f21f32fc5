"""Configuration: keys, defaults and refusals as the reference's parser has them
(src/loader/hf_checkpoint.cpp:28-136), the registry, and the translation into parts."""
import json

import pytest

from geneinfer_amd.config import (AttentionSpec, ConfigError, Llama3Scaling, LlamaConfig, ModelSpec, RunEntry, config_class_for,
                                  parse_config, read_config, register_architecture, registered_architectures)
from model_folders import CONFIGS, full_config

REQUIRED = dict(model_type="llama", hidden_size=64, intermediate_size=192, num_hidden_layers=2, num_attention_heads=4, vocab_size=256)


def test_only_required_keys_get_the_reference_defaults():
    c = parse_config({"model_type": "llama", **REQUIRED})          # tools/hf_io.py:105-120
    assert isinstance(c, LlamaConfig)
    assert (c.num_key_value_heads, c.head_dim, c.max_position_embeddings) == (4, 16, 2048)
    assert c.rope_theta == 10000.0 and c.rms_norm_eps == 1e-6 and c.rope_scaling is None and c.tie_word_embeddings is False
    assert c.attn_dim == 64 and c.kv_dim == 64


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_every_size_comes_from_the_file(name):
    sizes = CONFIGS[name]
    c = parse_config(full_config(sizes))
    for key in ("hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads", "vocab_size",
                "rope_theta", "rms_norm_eps", "tie_word_embeddings", "max_position_embeddings"):
        assert getattr(c, key) == sizes[key]
    assert c.head_dim == sizes.get("head_dim", sizes["hidden_size"] // sizes["num_attention_heads"])
    if sizes["rope_scaling"]:
        s = sizes["rope_scaling"]
        assert c.rope_scaling == Llama3Scaling(s["factor"], s["low_freq_factor"], s["high_freq_factor"], s["original_max_position_embeddings"])
    assert parse_config(json.loads(c.to_json())) == c                # what it writes reads back equal


def test_head_dim_may_differ_from_hidden_over_heads():
    c = parse_config({**REQUIRED, "hidden_size": 48, "head_dim": 16})
    assert c.attn_dim == 64 and c.hidden_size == 48
    spec = c.model_spec()
    assert spec.layers[0].mixer.head_dim == 16 and spec.layers[0].mixer.hidden_size == 48
    assert parse_config({**REQUIRED, "head_dim": None}).head_dim == 16      # null counts as absent


@pytest.mark.parametrize("change,message", [
    ({"hidden_size": None}, "has no 'hidden_size'"), ({"vocab_size": 0}, "'vocab_size' has an invalid value"),
    ({"num_hidden_layers": 2.5}, "invalid value"), ({"model_type": "mistral"}, "unknown architecture .model_type 'mistral'"), ({"architectures": ["LlamaForCausalLM"], "model_type": "qwen3"}, "unsupported model_type 'qwen3'"),
    ({"hidden_act": "gelu"}, "unsupported hidden_act"), ({"attention_bias": True}, "attention_bias = true"),
    ({"mlp_bias": True}, "mlp_bias = true"), ({"num_attention_heads": 5}, "not divisible by num_attention_heads"),
    ({"num_key_value_heads": 3}, "divisible by num_key_value_heads"), ({"head_dim": 15}, "head_dim must be even"),
    ({"rope_scaling": []}, "not an object"), ({"rope_scaling": {"rope_type": "yarn", "factor": 2}}, "'yarn' is not supported"),
    ({"rope_scaling": {"factor": 2}}, "is not supported"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 2, "low_freq_factor": 1, "high_freq_factor": 4}}, "original_max_position_embeddings is required"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 0.5, "low_freq_factor": 1, "high_freq_factor": 4, "original_max_position_embeddings": 64}}, "factor must be >= 1"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 8, "low_freq_factor": 4, "high_freq_factor": 4, "original_max_position_embeddings": 64}}, "0 < low_freq_factor < high_freq_factor"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 8, "low_freq_factor": 1, "high_freq_factor": 4, "original_max_position_embeddings": 0}}, "positive integer"),
])
def test_refusals_name_the_key(change, message):                     # tests/verify_hf_loader.py:203-227
    cfg = {"model_type": "llama", **REQUIRED, **change}
    cfg = {k: v for k, v in cfg.items() if v is not None}
    with pytest.raises(ConfigError, match=message):
        parse_config(cfg)


def test_rope_scaling_default_and_null_mean_none():
    for s in (None, {"rope_type": "default"}, {"type": "default", "factor": 3}):
        assert parse_config({**REQUIRED, "rope_scaling": s}).rope_scaling is None
    s = parse_config({**REQUIRED, "rope_scaling": {"type": "llama3", "factor": 8, "low_freq_factor": 1, "high_freq_factor": 4,
                                                   "original_max_position_embeddings": 8192}}).rope_scaling
    assert s == Llama3Scaling(8.0, 1.0, 4.0, 8192)


def test_registry_chooses_by_architecture_then_model_type():
    assert config_class_for({"architectures": ["LlamaForCausalLM"]}) is LlamaConfig
    assert config_class_for({"model_type": "llama"}) is LlamaConfig
    with pytest.raises(ConfigError, match=r"unknown architecture 'FooForCausalLM'; registered: .*LlamaForCausalLM"):
        parse_config({"architectures": ["FooForCausalLM"], **REQUIRED})
    with pytest.raises(ConfigError, match="unknown architecture"):
        parse_config({k: v for k, v in REQUIRED.items() if k != "model_type"})      # neither key names one


def test_another_architecture_registers_without_touching_the_framework():
    class Other:
        @classmethod
        def from_dict(cls, d):
            return cls()

    register_architecture("OtherForCausalLM", Other, model_type="other")
    assert "OtherForCausalLM" in registered_architectures()
    assert isinstance(parse_config({"model_type": "other"}), Other)
    with pytest.raises(ValueError, match="already registered"):
        register_architecture("OtherForCausalLM", LlamaConfig)


def test_read_config_errors(tmp_path):
    with pytest.raises(ConfigError, match="no config.json"):
        read_config(tmp_path)
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="config.json:"):
        read_config(tmp_path)


def test_model_spec_names_and_shapes():
    c = parse_config(full_config(CONFIGS["B"]))
    spec = c.model_spec()
    assert isinstance(spec, ModelSpec) and len(spec.layers) == 3 and spec.run_order == tuple(RunEntry(i) for i in range(3))
    m = spec.layers[1].mixer
    assert isinstance(m, AttentionSpec) and (m.n_heads, m.n_kv_heads, m.head_dim, m.window) == (3, 1, 32, None)
    assert m.q_proj == "model.layers.1.self_attn.q_proj.weight" and c.rope_scaling.factor == 4.0
    # the neutral spec carries the frequencies the architecture's rule has made: the first as theta gives it, the last a quarter of it
    f = m.position.frequencies
    assert len(f) == 16 and f[0] == 1.0 and abs(f[-1] * 4.0 * 500000.0 ** (30 / 32) - 1.0) < 1e-12
    assert parse_config(full_config(CONFIGS["A"])).model_spec().layers[0].mixer.position.frequencies is None
    assert spec.lm_head == "lm_head.weight" and spec.embedding == "model.embed_tokens.weight"
    tied = parse_config(full_config(CONFIGS["A"])).model_spec()
    assert tied.lm_head == tied.embedding and any("lm_head" in p for p in tied.ignorable_tensors)


def test_run_order_is_checked():
    spec = parse_config(full_config(CONFIGS["A"])).model_spec()
    import dataclasses
    with pytest.raises(ValueError, match="names layer 5"):
        dataclasses.replace(spec, run_order=(RunEntry(0), RunEntry(5)))
    with pytest.raises(ValueError, match="does not run before"):
        dataclasses.replace(spec, run_order=(RunEntry(0, cache_of=1), RunEntry(1)))
    twice = dataclasses.replace(spec, run_order=(RunEntry(0), RunEntry(1), RunEntry(0), RunEntry(1, cache_of=1)))
    assert len(twice.run_order) == 4                                 # a layer named twice, a layer reading another's cache
