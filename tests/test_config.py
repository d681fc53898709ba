"""Configuration parsing and the architecture registry.

Vectors from the reference's tests/unit/model/test_config_and_loader.py:16-89.
"""

from __future__ import annotations

import json

import pytest

import dli_amd.architectures  # noqa: F401
from dli_amd.config import (
    ConfigError, LlamaConfig, MissingConfigKeyError, UnsupportedModelError, load_config,
    register_architecture, registered_architectures, resolve_architecture, unregister_architecture,
)
from tiny_configs import TINY_A, TINY_B, TINY_C

HUB_LLAMA = {  # hub-style config.json with the old rope keys
    "model_type": "llama", "vocab_size": 49152, "hidden_size": 576, "intermediate_size": 1536,
    "num_hidden_layers": 30, "num_attention_heads": 9, "num_key_value_heads": 3, "rms_norm_eps": 1e-5,
    "rope_theta": 100000, "rope_scaling": None, "tie_word_embeddings": True, "hidden_act": "silu",
}


def test_hub_config_defaults():
    cfg = LlamaConfig.from_hf_dict(HUB_LLAMA)
    assert (cfg.head_dim, cfg.num_queries_per_kv) == (64, 3)
    assert cfg.rope.theta == 100000 and cfg.rope.rope_type == "default"
    assert not cfg.qkv_bias and not cfg.o_bias and not cfg.mlp_bias
    assert cfg.max_position_embeddings == 4096
    assert cfg.tie_word_embeddings


def test_rope_parameters_win_and_legacy_type_key():
    v5 = LlamaConfig.from_hf_dict({**HUB_LLAMA, "rope_theta": None, "rope_parameters": {
        "rope_type": "llama3", "rope_theta": 5e5, "factor": 8.0, "original_max_position_embeddings": 8192}})
    assert (v5.rope.rope_type, v5.rope.theta, v5.rope.factor) == ("llama3", 5e5, 8.0)
    assert (v5.rope.low_freq_factor, v5.rope.high_freq_factor) == (1.0, 4.0)
    legacy = LlamaConfig.from_hf_dict({**HUB_LLAMA, "rope_scaling": {"type": "linear", "factor": 2}})
    assert legacy.rope.rope_type == "linear" and legacy.rope.factor == 2.0
    both = LlamaConfig.from_hf_dict({**HUB_LLAMA, "rope_scaling": {"rope_type": "linear", "factor": 2},
                                     "rope_parameters": {"rope_type": "llama3", "factor": 4.0}})
    assert both.rope.rope_type == "llama3" and both.rope.factor == 4.0
    # llama3 without its own original length falls back to max_position_embeddings
    fb = LlamaConfig.from_hf_dict({**HUB_LLAMA, "max_position_embeddings": 2048,
                                   "rope_scaling": {"rope_type": "llama3", "factor": 8.0}})
    assert fb.rope.original_max_position_embeddings == 2048


@pytest.mark.parametrize("override", [
    {"model_type": "mistral"}, {"hidden_act": "gelu"}, {"use_sliding_window": True},
    {"layer_types": ["full_attention", "sliding_attention"]},
    {"rope_scaling": {"rope_type": "yarn", "factor": 4.0}}, {"pretraining_tp": 2},
    {"num_key_value_heads": 4},  # 9 heads do not group onto 4
    {"head_dim": 63},
])
def test_unsupported_features_are_refused(override):
    with pytest.raises(UnsupportedModelError):
        LlamaConfig.from_hf_dict({**HUB_LLAMA, **override})


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                                 "num_attention_heads", "rms_norm_eps"])
def test_keys_without_default_are_required(key):
    cfg = {k: v for k, v in HUB_LLAMA.items() if k != key}
    with pytest.raises(MissingConfigKeyError) as exc:
        LlamaConfig.from_hf_dict(cfg)
    assert key in str(exc.value)
    assert isinstance(exc.value, KeyError) and isinstance(exc.value, ConfigError)


def test_scaled_rope_needs_its_factor():
    with pytest.raises(MissingConfigKeyError):
        LlamaConfig.from_hf_dict({**HUB_LLAMA, "rope_scaling": {"rope_type": "linear"}})


@pytest.mark.parametrize("raw", [TINY_A, TINY_B, TINY_C, HUB_LLAMA])
def test_round_trip_through_config_json(raw, tmp_path):
    cfg = LlamaConfig.from_hf_dict(raw)
    again = LlamaConfig.from_hf_dict(cfg.to_hf_dict())
    assert again == cfg
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_hf_dict()))
    assert load_config(tmp_path) == cfg


def test_parameter_count_formula():
    # Llama-3.2-1B: 1,235,814,400 parameters
    cfg = LlamaConfig.from_hf_dict({
        "model_type": "llama", "vocab_size": 128256, "hidden_size": 2048, "intermediate_size": 8192,
        "num_hidden_layers": 16, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 64,
        "rms_norm_eps": 1e-5, "tie_word_embeddings": True})
    assert cfg.num_parameters() == 1_235_814_400


def test_registry_resolves_by_architecture_then_model_type():
    assert "LlamaForCausalLM" in registered_architectures()
    assert resolve_architecture({"architectures": ["LlamaForCausalLM"]}).name == "LlamaForCausalLM"
    assert resolve_architecture({"model_type": "llama"}).name == "LlamaForCausalLM"
    with pytest.raises(UnsupportedModelError, match="Mystery"):
        resolve_architecture({"architectures": ["MysteryForCausalLM"], "model_type": "llama"})
    with pytest.raises(UnsupportedModelError):
        resolve_architecture({"model_type": "qwen2"})


def test_another_architecture_registers_without_touching_the_framework():
    seen = {}
    register_architecture("ToyForCausalLM", lambda raw: {"parsed": raw["width"]},
                          lambda cfg: seen.setdefault("spec", cfg), model_types=("toy",))
    try:
        arch = resolve_architecture({"architectures": ["ToyForCausalLM"], "width": 8})
        assert arch.build_spec(arch.parse_config({"width": 8})) == {"parsed": 8}
        with pytest.raises(ConfigError, match="already"):
            register_architecture("ToyForCausalLM", dict, dict)
    finally:
        unregister_architecture("ToyForCausalLM")
    assert "ToyForCausalLM" not in registered_architectures()


def test_config_json_problems_are_clear(tmp_path):
    with pytest.raises(ConfigError, match="does not exist"):
        load_config(tmp_path)
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="not valid JSON"):
        load_config(tmp_path)
