"""Typed configuration of the dense Llama decoder (Llama 3.2, SmolLM2).

Every size and constant of the model is a field here, read from the architecture's own
``config.json`` keys; nothing below this module carries a literal size.
Parsing rules follow the reference's ``ModelConfig.from_hf_dict`` (src/dli/model/config.py:80-150).
"""

from __future__ import annotations

from dataclasses import dataclass, fields
from typing import Any, Mapping

from .errors import MissingConfigKeyError, UnsupportedModelError

SUPPORTED_ROPE_TYPES = ("default", "linear", "llama3")


@dataclass(frozen=True)
class RopeConfig:
    """Rotary position encoding constants (reference: src/dli/model/config.py:22-39).

    ``rope_type`` is ``default`` (plain geometric frequencies), ``linear`` (all frequencies divided
    by ``factor``) or ``llama3`` (low frequencies divided by ``factor``, high ones kept, a smooth
    blend between, bands measured against ``original_max_position_embeddings``).
    """

    theta: float
    rope_type: str = "default"
    factor: float = 1.0
    low_freq_factor: float = 1.0
    high_freq_factor: float = 4.0
    original_max_position_embeddings: int = 8192

    def __post_init__(self) -> None:
        if self.rope_type not in SUPPORTED_ROPE_TYPES:
            raise UnsupportedModelError(f"rope_type={self.rope_type!r} is not supported")
        if not self.theta > 0:
            raise UnsupportedModelError(f"rope_theta={self.theta} must be positive")
        if self.rope_type != "default" and not self.factor > 0:
            raise UnsupportedModelError(f"rope factor={self.factor} must be positive")
        if self.rope_type == "llama3" and self.high_freq_factor == self.low_freq_factor:
            raise UnsupportedModelError("llama3 rope needs high_freq_factor != low_freq_factor")


@dataclass(frozen=True)
class LlamaConfig:
    """Hyper-parameters of ``LlamaForCausalLM`` (reference: src/dli/model/config.py:42-78)."""

    model_type: str
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    rms_norm_eps: float
    max_position_embeddings: int
    rope: RopeConfig
    tie_word_embeddings: bool
    hidden_act: str = "silu"
    qkv_bias: bool = False
    o_bias: bool = False
    mlp_bias: bool = False

    architecture = "LlamaForCausalLM"

    def __post_init__(self) -> None:
        for name in ("vocab_size", "hidden_size", "intermediate_size", "num_layers", "num_heads",
                     "num_kv_heads", "head_dim"):
            if getattr(self, name) < 1:
                raise UnsupportedModelError(f"{name}={getattr(self, name)} must be positive")
        if self.num_heads % self.num_kv_heads != 0:
            raise UnsupportedModelError(
                f"num_attention_heads={self.num_heads} is not a multiple of "
                f"num_key_value_heads={self.num_kv_heads}"
            )
        if self.head_dim % 2 != 0:
            raise UnsupportedModelError(f"head_dim={self.head_dim} must be even for RoPE")
        if not self.rms_norm_eps >= 0:
            raise UnsupportedModelError(f"rms_norm_eps={self.rms_norm_eps} must not be negative")

    @property
    def num_queries_per_kv(self) -> int:
        """Query heads that share one key/value head."""
        return self.num_heads // self.num_kv_heads

    def num_parameters(self) -> int:
        """Count of stored parameters (biases excluded unless configured)."""
        h, d = self.hidden_size, self.head_dim
        q, kv, inter = self.num_heads * d, self.num_kv_heads * d, self.intermediate_size
        per_layer = h * q + 2 * h * kv + q * h + 3 * h * inter + 2 * h
        if self.qkv_bias:
            per_layer += q + 2 * kv
        if self.o_bias:
            per_layer += h
        if self.mlp_bias:
            per_layer += 2 * inter + h
        head = self.vocab_size * h * (1 if self.tie_word_embeddings else 2)
        return self.num_layers * per_layer + head + h

    @classmethod
    def from_hf_dict(cls, cfg: Mapping[str, Any]) -> "LlamaConfig":
        """Parse a ``config.json`` dictionary.

        Accepts the hub spelling (``rope_theta`` + ``rope_scaling``) and the newer
        ``rope_parameters`` one (which wins where both are present).

        Raises:
            UnsupportedModelError: another architecture, or an option that is not implemented.
            MissingConfigKeyError: a key without default is absent.
        """
        model_type = cfg.get("model_type")
        if model_type != "llama":
            raise UnsupportedModelError(f"model_type={model_type!r} is not supported")
        act = cfg.get("hidden_act", "silu")
        if act != "silu":
            raise UnsupportedModelError(f"hidden_act={act!r} (only 'silu' / SwiGLU is supported)")
        if cfg.get("use_sliding_window") or any(
            t != "full_attention" for t in cfg.get("layer_types") or []
        ):
            raise UnsupportedModelError("sliding-window attention is not supported")
        if cfg.get("pretraining_tp", 1) not in (1, None):
            raise UnsupportedModelError("pretraining_tp > 1 changes numerics and is not supported")

        def need(key: str) -> Any:
            if cfg.get(key) is None:
                raise MissingConfigKeyError(key)
            return cfg[key]

        num_heads = int(need("num_attention_heads"))
        hidden = int(need("hidden_size"))
        attention_bias = bool(cfg.get("attention_bias", False))
        return cls(
            model_type=model_type,
            vocab_size=int(need("vocab_size")),
            hidden_size=hidden,
            intermediate_size=int(need("intermediate_size")),
            num_layers=int(need("num_hidden_layers")),
            num_heads=num_heads,
            num_kv_heads=int(cfg.get("num_key_value_heads") or num_heads),
            head_dim=int(cfg.get("head_dim") or hidden // num_heads),
            rms_norm_eps=float(need("rms_norm_eps")),
            max_position_embeddings=int(cfg.get("max_position_embeddings", 4096)),
            rope=_parse_rope(cfg),
            tie_word_embeddings=bool(cfg.get("tie_word_embeddings", False)),
            hidden_act=act,
            qkv_bias=attention_bias,
            o_bias=attention_bias,
            mlp_bias=bool(cfg.get("mlp_bias", False)),
        )

    def to_hf_dict(self) -> dict[str, Any]:
        """The ``config.json`` dictionary that parses back to this configuration."""
        out: dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": self.model_type,
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_layers,
            "num_attention_heads": self.num_heads,
            "num_key_value_heads": self.num_kv_heads,
            "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps,
            "max_position_embeddings": self.max_position_embeddings,
            "rope_theta": self.rope.theta,
            "rope_scaling": None,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": self.hidden_act,
            "attention_bias": self.qkv_bias,
            "mlp_bias": self.mlp_bias,
        }
        if self.qkv_bias != self.o_bias:
            raise UnsupportedModelError("config.json has one attention_bias flag for q, k, v and o")
        if self.rope.rope_type != "default":
            scaling: dict[str, Any] = {"rope_type": self.rope.rope_type, "factor": self.rope.factor}
            if self.rope.rope_type == "llama3":
                scaling.update(
                    low_freq_factor=self.rope.low_freq_factor,
                    high_freq_factor=self.rope.high_freq_factor,
                    original_max_position_embeddings=self.rope.original_max_position_embeddings,
                )
            out["rope_scaling"] = scaling
        return out


def _parse_rope(cfg: Mapping[str, Any]) -> RopeConfig:
    """Rotary constants from either spelling (reference: src/dli/model/config.py:130-150)."""
    merged: dict[str, Any] = {**dict(cfg.get("rope_scaling") or {}),
                              **dict(cfg.get("rope_parameters") or {})}
    theta = merged.get("rope_theta")
    if theta is None:
        theta = cfg.get("rope_theta")
    if theta is None:
        theta = 10000.0
    rope_type = merged.get("rope_type", merged.get("type", "default"))
    if rope_type not in SUPPORTED_ROPE_TYPES:
        raise UnsupportedModelError(f"rope_type={rope_type!r} is not supported")
    if rope_type == "default":
        return RopeConfig(theta=float(theta))
    if merged.get("factor") is None:
        raise MissingConfigKeyError("rope_scaling.factor")
    return RopeConfig(
        theta=float(theta),
        rope_type=rope_type,
        factor=float(merged["factor"]),
        low_freq_factor=float(merged.get("low_freq_factor", 1.0)),
        high_freq_factor=float(merged.get("high_freq_factor", 4.0)),
        original_max_position_embeddings=int(
            merged.get("original_max_position_embeddings", cfg.get("max_position_embeddings", 8192))
        ),
    )


def config_field_names() -> tuple[str, ...]:
    return tuple(f.name for f in fields(LlamaConfig))
