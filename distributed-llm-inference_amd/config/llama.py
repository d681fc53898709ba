"""Typed configuration of the dense Llama decoder (Llama 3.2, SmolLM2).

Every size and constant of the model is a field here, read from the architecture's own
``config.json`` keys; nothing below this module carries a literal size.
What is read, defaulted and refused is what the reference's ``ModelConfig.from_hf_dict`` reads,
defaults and refuses (src/dli/model/config.py:80-150).
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
        """Parse a ``config.json`` dictionary: refusals first (:data:`_REFUSALS`), then every
        field from its key by :data:`_FIELDS`, then the rotary constants from whichever of the two
        spellings the file uses (``rope_theta`` + ``rope_scaling``, or ``rope_parameters``).

        Raises:
            UnsupportedModelError: another architecture, or an option that is not implemented.
            MissingConfigKeyError: a key without default is absent.
        """
        for refused, why in _REFUSALS:
            if refused(cfg):
                raise UnsupportedModelError(why(cfg))
        values: dict[str, Any] = {}
        for name, key, cast, default in _FIELDS:
            raw = cfg.get(key)
            if raw is None:
                if default is _REQUIRED:
                    raise MissingConfigKeyError(key)
                raw = default(values) if callable(default) else default
            values[name] = cast(raw)
        bias = values.pop("attention_bias")  # one flag in the file, two places in the model
        return cls(rope=_read_rope(cfg), qkv_bias=bias, o_bias=bias, **values)

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


_REQUIRED = object()

# What is refused before anything is read: (test on the dictionary, message).
_REFUSALS = (
    (lambda c: c.get("model_type") != "llama",
     lambda c: f"model_type {c.get('model_type')!r}: this configuration reads 'llama' only"),
    (lambda c: c.get("hidden_act", "silu") != "silu",
     lambda c: f"hidden_act {c.get('hidden_act')!r}: the feed-forward is gated with SiLU and nothing else"),
    (lambda c: bool(c.get("use_sliding_window")) or any(t != "full_attention" for t in c.get("layer_types") or ()),
     lambda c: "layers with a sliding window are not part of this architecture here"),
    (lambda c: (c.get("pretraining_tp") or 1) != 1,
     lambda c: f"pretraining_tp {c.get('pretraining_tp')}: products cut in slices round differently; only 1 is taken"),
)

# field, config.json key, type, default (a value, a function of the fields read so far, or required)
_FIELDS = (
    ("model_type", "model_type", str, _REQUIRED),
    ("vocab_size", "vocab_size", int, _REQUIRED),
    ("hidden_size", "hidden_size", int, _REQUIRED),
    ("intermediate_size", "intermediate_size", int, _REQUIRED),
    ("num_layers", "num_hidden_layers", int, _REQUIRED),
    ("num_heads", "num_attention_heads", int, _REQUIRED),
    ("num_kv_heads", "num_key_value_heads", int, lambda v: v["num_heads"]),
    ("head_dim", "head_dim", int, lambda v: v["hidden_size"] // v["num_heads"]),
    ("rms_norm_eps", "rms_norm_eps", float, _REQUIRED),
    ("max_position_embeddings", "max_position_embeddings", int, 4096),
    ("tie_word_embeddings", "tie_word_embeddings", bool, False),
    ("hidden_act", "hidden_act", str, "silu"),
    ("attention_bias", "attention_bias", bool, False),
    ("mlp_bias", "mlp_bias", bool, False),
)


def _read_rope(cfg: Mapping[str, Any]) -> RopeConfig:
    """Rotary constants (reference: src/dli/model/config.py:130-150). A constant is looked up in
    ``rope_parameters`` first, then in ``rope_scaling``, then (theta only) at the top level; old
    files call the type ``type``."""
    places = [cfg.get("rope_parameters") or {}, cfg.get("rope_scaling") or {}]

    def find(*keys: str, top_level: bool = False, default: Any = None) -> Any:
        for place in places + ([cfg] if top_level else []):
            for key in keys:
                if place.get(key) is not None:
                    return place[key]
        return default

    theta = float(find("rope_theta", top_level=True, default=10000.0))
    kind = find("rope_type", "type", default="default")
    if kind == "default":
        return RopeConfig(theta=theta)
    if kind not in SUPPORTED_ROPE_TYPES:
        raise UnsupportedModelError(f"rope_type {kind!r}: one of {SUPPORTED_ROPE_TYPES} is needed")
    factor = find("factor")
    if factor is None:
        raise MissingConfigKeyError("rope_scaling.factor")
    return RopeConfig(
        theta=theta, rope_type=kind, factor=float(factor),
        low_freq_factor=float(find("low_freq_factor", default=1.0)),
        high_freq_factor=float(find("high_freq_factor", default=4.0)),
        original_max_position_embeddings=int(find(
            "original_max_position_embeddings", default=cfg.get("max_position_embeddings") or 8192)))


def config_field_names() -> tuple[str, ...]:
    return tuple(f.name for f in fields(LlamaConfig))
