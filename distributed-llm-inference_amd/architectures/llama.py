"""``LlamaForCausalLM``: the dense Llama decoder (Llama 3.2, SmolLM2) as a list of parts.

Tensor names are the checkpoint's own (reference: src/dli/model/llama.py:5-6,216-247):
``model.embed_tokens.weight``, ``model.layers.{i}.input_layernorm.weight``,
``model.layers.{i}.self_attn.{q,k,v,o}_proj.weight``, ``model.layers.{i}.post_attention_layernorm
.weight``, ``model.layers.{i}.mlp.{gate,up,down}_proj.weight``, ``model.norm.weight`` and, when the
head is not tied to the embedding, ``lm_head.weight``.
"""

from __future__ import annotations

from ..config.llama import LlamaConfig
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


def build_llama_spec(cfg: LlamaConfig) -> ModelSpec:
    rope = cfg.rope
    position = PartSpec("rotary", dict(
        dim=cfg.head_dim, theta=rope.theta, rope_type=rope.rope_type, factor=rope.factor,
        low_freq_factor=rope.low_freq_factor, high_freq_factor=rope.high_freq_factor,
        original_max_position_embeddings=rope.original_max_position_embeddings))
    norm = dict(width=cfg.hidden_size, eps=cfg.rms_norm_eps)
    layers = []
    for i in range(cfg.num_layers):
        p = f"model.layers.{i}."
        layers.append(LayerSpec(
            block=PartSpec("pre_norm"),
            parts={
                "mixer_norm": ("norm", PartSpec("rms_norm", norm, p + "input_layernorm.")),
                "mixer": ("mixer", PartSpec("gqa_attention", dict(
                    hidden_size=cfg.hidden_size, num_heads=cfg.num_heads, num_kv_heads=cfg.num_kv_heads,
                    head_dim=cfg.head_dim, position=position, qkv_bias=cfg.qkv_bias, o_bias=cfg.o_bias),
                    p + "self_attn.")),
                "feed_forward_norm": ("norm", PartSpec("rms_norm", norm, p + "post_attention_layernorm.")),
                "feed_forward": ("feed_forward", PartSpec("gated_mlp", dict(
                    hidden_size=cfg.hidden_size, intermediate_size=cfg.intermediate_size,
                    activation=cfg.hidden_act, bias=cfg.mlp_bias), p + "mlp.")),
            }))
    return ModelSpec(
        architecture=cfg.architecture,
        vocab_size=cfg.vocab_size,
        hidden_size=cfg.hidden_size,
        embedding=PartSpec("token_embedding", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size),
                           "model.embed_tokens."),
        layers=tuple(layers),
        schedule=tuple(ScheduleEntry(i) for i in range(cfg.num_layers)),
        final_norm=PartSpec("rms_norm", norm, "model.norm."),
        head=PartSpec("linear_head", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size,
                                          tied=cfg.tie_word_embeddings), "lm_head."),
        tied_aliases={"lm_head.weight": "model.embed_tokens.weight"} if cfg.tie_word_embeddings else {},
    )


register_architecture("LlamaForCausalLM", LlamaConfig.from_hf_dict, build_llama_spec,
                      model_types=("llama",), replace=True)
