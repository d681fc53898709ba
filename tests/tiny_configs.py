"""Two tiny Llama configurations that differ in every size and option, and model folders for them."""

from __future__ import annotations

import tempfile
from pathlib import Path

# 2 layers, MHA, head_dim 16, default rope, tied head, eps 1e-5
TINY_A = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "vocab_size": 256, "hidden_size": 64,
    "intermediate_size": 160, "num_hidden_layers": 2, "num_attention_heads": 4, "num_key_value_heads": 4,
    "head_dim": 16, "rms_norm_eps": 1e-5, "max_position_embeddings": 256, "rope_theta": 10000.0,
    "tie_word_embeddings": True, "hidden_act": "silu",
}
# 3 layers, GQA 3:1, head_dim 32, llama3 rope, untied head, eps 1e-6, widths no power of two
TINY_B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "vocab_size": 384, "hidden_size": 192,
    "intermediate_size": 512, "num_hidden_layers": 3, "num_attention_heads": 6, "num_key_value_heads": 2,
    "head_dim": 32, "rms_norm_eps": 1e-6, "max_position_embeddings": 512, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 64},
    "tie_word_embeddings": False, "hidden_act": "silu",
}
# odd sizes everywhere: 5 heads of 48 on a width of 200 (head_dim given, not hidden/heads),
# biases, linear rope, vocabulary 301
TINY_C = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "vocab_size": 301, "hidden_size": 200,
    "intermediate_size": 136, "num_hidden_layers": 2, "num_attention_heads": 5, "num_key_value_heads": 1,
    "head_dim": 48, "rms_norm_eps": 1e-5, "max_position_embeddings": 1024, "rope_theta": 10000.0,
    "rope_scaling": {"type": "linear", "factor": 2.0}, "attention_bias": True, "mlp_bias": True,
    "tie_word_embeddings": False, "hidden_act": "silu",
}
# the layer sizes of Llama-3.2-1B (width 2048, 32 heads of 64 on 8 kv heads, feed-forward 8192,
# llama3 rope, tied head) with two layers and a quarter of the vocabulary (odd on purpose): the
# kernels meet the shapes they serve
WIDE = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "vocab_size": 32003, "hidden_size": 2048,
    "intermediate_size": 8192, "num_hidden_layers": 2, "num_attention_heads": 32, "num_key_value_heads": 8,
    "head_dim": 64, "rms_norm_eps": 1e-5, "max_position_embeddings": 131072, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 8192},
    "tie_word_embeddings": True, "hidden_act": "silu",
}
# sizes that tile (width and feed-forward multiples of 128, vocabulary a multiple of 16): decode
# steps read the tile-ordered copies of the weights and rotate in the q/k/v product, as at the
# serving sizes, but on a model small enough for every way of cutting and batching
TINY_D = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "vocab_size": 512, "hidden_size": 256,
    "intermediate_size": 384, "num_hidden_layers": 2, "num_attention_heads": 8, "num_key_value_heads": 2,
    "head_dim": 32, "rms_norm_eps": 1e-5, "max_position_embeddings": 2048, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 4.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 128},
    "attention_bias": True, "tie_word_embeddings": True, "hidden_act": "silu",
}
# heads of 128 (the head size of Llama-3.2-3B) in groups of three on one and two kv heads' worth of
# width: the projections are wider than the model (6 x 128 on a width of 384), vocabulary odd
TINY_H = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "vocab_size": 331, "hidden_size": 384,
    "intermediate_size": 640, "num_hidden_layers": 2, "num_attention_heads": 6, "num_key_value_heads": 2,
    "head_dim": 128, "rms_norm_eps": 1e-5, "max_position_embeddings": 4096, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 256},
    "tie_word_embeddings": True, "hidden_act": "silu",
}
# Llama-3.2-1B as config.json has it: every layer and the whole vocabulary
LLAMA_3_2_1B = dict(WIDE, vocab_size=128256, num_hidden_layers=16)
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D, "H": TINY_H, "W": WIDE, "1B": LLAMA_3_2_1B}

_made: dict = {}
_tmp = None


# Weights are drawn with std = 1.2 / sqrt(hidden) instead of the usual 0.02: attention scores then
# have a spread of about one, so attention is far from uniform (a key in the wrong place, a wrong
# rotation or a wrong mask changes the logits) without being so sharp that bfloat16's rounding of a
# score is blown up into a different distribution.
STD = {"A": 0.15, "B": 0.085, "C": 0.085, "D": 0.075, "H": 0.06, "W": 0.0265, "1B": 0.0265}


def model_folder(name: str, seed: int = 11, std: float | None = None, norm_jitter: float = 0.1,
                 device: str = "cpu") -> Path:
    """A temporary folder with config.json and model.safetensors of configuration ``name``."""
    from dli_amd.weights import write_random_model

    global _tmp
    std = STD[name] if std is None else std
    key = (name, seed, std, norm_jitter, device)
    if key not in _made:
        if _tmp is None:
            _tmp = tempfile.TemporaryDirectory(prefix="dli_amd_tiny_")
        out = Path(_tmp.name) / f"{name}_{seed}_{std}_{norm_jitter}_{device}"
        write_random_model(out, CONFIGS[name], seed=seed, std=std, norm_jitter=norm_jitter, device=device)
        _made[key] = out
    return _made[key]
