"""Parts that models are put together from, their registry and the model assembled from a spec."""

from .base import (
    Block, CompositeCacheSpec, Embedding, FeedForward, Head, Mixer, Norm, PagedKVSpec, Part, PositionEncoding, RotaryTable, Runtime, StateSpec,
)
from .registry import build_part, part_class, register_part, registered_parts, unregister_part
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, WeightSpec

__all__ = [
    "Block", "CompositeCacheSpec", "Embedding", "FeedForward", "Head", "LayerSpec", "Mixer", "ModelSpec", "Norm", "PagedKVSpec",
    "Part", "PartSpec", "PositionEncoding", "RotaryTable", "Runtime", "ScheduleEntry", "StateSpec", "WeightSpec",
    "build_part", "part_class", "register_part", "registered_parts", "unregister_part",
]

# importing the modules registers the parts that ship with the engine
from . import (  # noqa: E402,F401
    attention, block, embedding, experts, feed_forward, head, norm, parallel, position, recurrent, scored_attention,
)
