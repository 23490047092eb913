from .registry import (register_reentry, register_mixer, register_feed_forward, register_norm, register_position,
                       register_embedding, register_head, register_arrangement, register_convolution, register_residual_gate, register_stream, register_connection, lookup,
                       registered)
from .base import Part, KVCacheSpec, PagedSpec, StateSpec
from . import norm, scalar_norm, rope, attention, hgrn2, latent_attention, short_conv, mlp, embedding, block, conv_attention, reentry, linear_attention, pooled_attention, residual_gate, hyper_connection, rglru, parallel_mixers  # noqa: F401  (register the built-in kinds)
from .model import DecoderModel, build_model, StepContext, KVView, StateView

__all__ = ["register_mixer", "register_feed_forward", "register_norm", "register_position",
           "register_embedding", "register_head", "register_arrangement", "register_convolution", "register_residual_gate", "register_stream", "register_connection", "lookup", "registered", "Part",
           "KVCacheSpec", "PagedSpec", "StateSpec", "DecoderModel", "build_model", "StepContext", "KVView", "StateView"]
