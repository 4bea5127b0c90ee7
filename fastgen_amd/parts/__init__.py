from .base import (
    MATRIX,
    TABLE_INT,
    VECTOR,
    FeedForward,
    LayerStore,
    Mixer,
    Norm,
    PagedNeed,
    Part,
    PositionEncoding,
    StateNeed,
    TensorSpec,
    build_part,
    place,
    register_part,
    registered_parts,
    unregister_part,
)
from . import attention, block, embedding, feed_forward, norm, position  # register the built-in parts

__all__ = [
    "MATRIX", "TABLE_INT", "VECTOR", "FeedForward", "LayerStore", "Mixer", "Norm", "PagedNeed", "Part",
    "PositionEncoding", "StateNeed", "TensorSpec", "build_part", "place", "register_part",
    "registered_parts", "unregister_part",
]
