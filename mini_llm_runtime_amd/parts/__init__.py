"""Parts a layer is put together from, and the model that runs them."""

from . import (  # noqa: F401  (register the built-in kinds)
    attention, block, feed_forward, gated_linear_attention, latent_attention, matrix_memory, norm, pooled_attention,
    position, retention, short_conv, sigmoid_attention, side_by_side, token_input,
)
from .base import Block, FeedForward, Mixer, Norm, Part, PositionEncoding
from .context import KVView, StateView, StepContext
from .model import DecoderModel
from .registry import build_part, part_kinds, register_part, unregister_part
from .spec import LayerSpec, ModelSpec, OrderEntry, ParamSpec, PartSpec, WeightRule

__all__ = [
    "Block",
    "DecoderModel",
    "FeedForward",
    "KVView",
    "LayerSpec",
    "Mixer",
    "ModelSpec",
    "Norm",
    "OrderEntry",
    "ParamSpec",
    "Part",
    "PartSpec",
    "PositionEncoding",
    "StateView",
    "StepContext",
    "WeightRule",
    "build_part",
    "part_kinds",
    "register_part",
    "unregister_part",
]
