"""Parts that models are put together from, their registry and the model assembled from a spec."""

from .base import (
    Block, Embedding, FeedForward, Head, Mixer, Norm, PagedKVSpec, Part, PositionEncoding, RotaryTable, Runtime, StateSpec,
)
from .registry import build_part, part_class, register_part, registered_parts, unregister_part
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, WeightSpec

__all__ = [
    "Block", "Embedding", "FeedForward", "Head", "LayerSpec", "Mixer", "ModelSpec", "Norm", "PagedKVSpec",
    "Part", "PartSpec", "PositionEncoding", "RotaryTable", "Runtime", "ScheduleEntry", "StateSpec", "WeightSpec",
    "build_part", "part_class", "register_part", "registered_parts", "unregister_part",
]

# importing the modules registers the parts that ship with the engine
from . import attention, block, embedding, feed_forward, head, norm, position  # noqa: E402,F401
