from .base import (
    MATRIX,
    TABLE_INT,
    VECTOR,
    FeedForward,
    Injection,
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
from . import (attention, block, embedding, feed_forward, injection, latent_attention, linear_attention, moe, norm,  # noqa: F401
               position, selective_scan, sigmoid_attention)  # register the built-in parts

__all__ = [
    "MATRIX", "TABLE_INT", "VECTOR", "FeedForward", "Injection", "LayerStore", "Mixer", "Norm", "PagedNeed", "Part",
    "PositionEncoding", "StateNeed", "TensorSpec", "build_part", "place", "register_part",
    "registered_parts", "unregister_part",
]
