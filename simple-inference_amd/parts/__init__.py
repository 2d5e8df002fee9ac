from .plan import LayerSpec, ModelPlan, PagedKVNeed, PartSpec, StateNeed, TensorSpec
from .registry import (
    BLOCKS, EMBEDDINGS, FEED_FORWARDS, GATES, HEADS, MIXERS, NORMS, POSITION_ENCODINGS, STREAM_OPS,
    register_block, register_embedding, register_feed_forward, register_gate, register_head, register_mixer,
    register_norm, register_position_encoding, register_stream_op,
)
from .context import BiasedDelta, BuildEnv, LayerCache, ResidualStream, ScaledSum, StepContext
from . import norm, rope, attention, swiglu, dense, block, embedding, gate, stream_ops, gla, moe, ssm, hgrn, latent_attention, delta, decay_attention, parallel  # noqa: F401  (registers the built-in kinds)
from .model import DecoderModel

__all__ = [
    "LayerSpec", "ModelPlan", "PagedKVNeed", "PartSpec", "StateNeed", "TensorSpec",
    "BLOCKS", "EMBEDDINGS", "FEED_FORWARDS", "GATES", "HEADS", "MIXERS", "NORMS", "POSITION_ENCODINGS", "STREAM_OPS",
    "register_block", "register_embedding", "register_feed_forward", "register_gate", "register_head", "register_mixer",
    "register_norm", "register_position_encoding", "register_stream_op",
    "BiasedDelta", "BuildEnv", "LayerCache", "ResidualStream", "ScaledSum", "StepContext", "DecoderModel",
]
