"""The data that describes a model: which parts it is made of, with which sizes, in which order.

A :class:`ModelSpec` is produced by an architecture's builder from its typed configuration and is
all that the rest of the engine knows about the model. It names parts by *family* and *kind*
(``mixer/gqa_attention``, ``feed_forward/swiglu``, ...) with their sizes and constants as plain
parameters; the part registry turns each :class:`PartSpec` into an object. Layers may differ from
one another, and the order in which they run is a list of its own (:class:`ScheduleEntry`): it may
name a layer twice (shared weights) or let an entry read the cache that another entry writes.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional


@dataclass(frozen=True)
class WeightSpec:
    """One tensor that a part binds, by its name below the part's prefix.

    ``role`` decides the stored type: ``"matrix"`` tensors take the engine's activation type
    (bfloat16 when serving, float32 on the 32-bit path); ``"float32"`` tensors are kept in 32-bit
    whatever the engine's type (norm weights, and anything a checkpoint stores in 32-bit on
    purpose); ``"int32"`` tensors are integer tables.
    """

    shape: tuple[int, ...]
    role: str = "matrix"
    optional: bool = False
    init: str = "normal"  # random-weights mode: "normal" (std 0.02), "ones", "zeros", "norm"

    def __post_init__(self) -> None:
        if self.role not in ("matrix", "float32", "int32"):
            raise ValueError(f"unknown weight role {self.role!r}")


@dataclass(frozen=True)
class PartSpec:
    """A part by family-specific ``kind`` with its parameters and checkpoint-name ``prefix``."""

    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)
    prefix: str = ""


@dataclass(frozen=True)
class LayerSpec:
    """One layer: a block arrangement and the parts it arranges, by role.

    The ``pre_norm`` arrangement uses the roles ``mixer_norm``, ``mixer``, ``feed_forward_norm``
    and ``feed_forward``; another arrangement may use others.
    """

    block: PartSpec
    parts: Mapping[str, tuple[str, PartSpec]]  # role -> (family, spec)


@dataclass(frozen=True)
class ScheduleEntry:
    """Run ``layer``. With ``cache_of`` the entry reads the cache that schedule entry ``cache_of``
    wrote earlier in the same step instead of keeping one of its own."""

    layer: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    embedding: PartSpec
    layers: tuple[LayerSpec, ...]
    schedule: tuple[ScheduleEntry, ...]
    final_norm: PartSpec
    head: PartSpec
    # checkpoint names that must equal another tensor when present, and are then dropped
    # (a tied model whose file still carries lm_head.weight): alias -> canonical name
    tied_aliases: Mapping[str, str] = field(default_factory=dict)

    def __post_init__(self) -> None:
        for i, e in enumerate(self.schedule):
            if not 0 <= e.layer < len(self.layers):
                raise ValueError(f"schedule entry {i} names layer {e.layer} of {len(self.layers)}")
            if e.cache_of is not None:
                if not 0 <= e.cache_of < i:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {e.cache_of}, "
                                     "which does not run before it")
                if self.schedule[e.cache_of].cache_of is not None:
                    raise ValueError(f"schedule entry {i} reads the cache of an entry that has none")
