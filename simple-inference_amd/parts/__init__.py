from .plan import LayerSpec, ModelPlan, PagedKVNeed, PartSpec, StateNeed, TensorSpec
from .registry import (
    BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS,
    register_block, register_embedding, register_feed_forward, register_head, register_mixer, register_norm,
    register_position_encoding,
)
from .context import BuildEnv, LayerCache, ResidualStream, StepContext
from . import norm, rope, attention, swiglu, block, embedding  # noqa: F401  (registers the built-in kinds)
from .model import DecoderModel

__all__ = [
    "LayerSpec", "ModelPlan", "PagedKVNeed", "PartSpec", "StateNeed", "TensorSpec",
    "BLOCKS", "EMBEDDINGS", "FEED_FORWARDS", "HEADS", "MIXERS", "NORMS", "POSITION_ENCODINGS",
    "register_block", "register_embedding", "register_feed_forward", "register_head", "register_mixer",
    "register_norm", "register_position_encoding",
    "BuildEnv", "LayerCache", "ResidualStream", "StepContext", "DecoderModel",
]
