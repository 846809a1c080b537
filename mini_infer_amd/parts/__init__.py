"""Parts a layer is put together from.  Importing this package registers the built-in kinds."""

from mini_infer_amd.parts import (  # noqa: F401
    attention, block, embedding, feed_forward, latent_attention, norm, position, recurrent, side_by_side,
)
from mini_infer_amd.parts.base import (
    Block,
    CacheNeeds,
    Embedding,
    FeedForward,
    Head,
    LayerCache,
    Mixer,
    Norm,
    PagedKVNeeds,
    ParamSpec,
    Part,
    PositionEncoding,
    RotaryTables,
    StateNeeds,
    StepContext,
)

__all__ = [
    "Block",
    "CacheNeeds",
    "Embedding",
    "FeedForward",
    "Head",
    "LayerCache",
    "Mixer",
    "Norm",
    "PagedKVNeeds",
    "ParamSpec",
    "Part",
    "PositionEncoding",
    "RotaryTables",
    "StateNeeds",
    "StepContext",
]
