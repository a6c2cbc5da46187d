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
from . import (attention, block, differential_attention, embedding, feed_forward, injection, latent_attention,  # noqa: F401
               linear_attention, moe, norm, position, selective_scan, sigmoid_attention)  # register the built-in parts

__all__ = [
    "MATRIX", "TABLE_INT", "VECTOR", "FeedForward", "Injection", "LayerStore", "Mixer", "Norm", "PagedNeed", "Part",
    "PositionEncoding", "StateNeed", "TensorSpec", "build_part", "place", "register_part",
    "registered_parts", "unregister_part",
]
