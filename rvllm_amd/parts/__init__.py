"""Parts of a layer and their registries.  Importing the package registers the
parts the framework ships."""

from . import (attention, block, delta_rule, embedding, experts, feedforward, latent_attention,  # noqa: F401
               linear_recurrence, matrix_memory, norm, rope, selective_scan, side_by_side)  # noqa: F401  (register themselves)
from .base import (Block, Embedding, FeedForward, Head, KVCacheView, KVNeed, Mixer, Norm, ParamSpec, Part,
                   PositionEncoding, StateNeed, StateView)
from .registry import BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

__all__ = [
    "Block", "Embedding", "FeedForward", "Head", "KVCacheView", "KVNeed", "Mixer", "Norm", "ParamSpec", "Part",
    "PositionEncoding", "StateNeed", "StateView", "BLOCKS", "EMBEDDINGS", "FEED_FORWARDS", "HEADS", "MIXERS", "NORMS",
    "POSITION_ENCODINGS", "LayerSpec", "ModelSpec", "PartSpec", "ScheduleEntry",
]
