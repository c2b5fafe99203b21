from .registry import (register_mixer, register_feed_forward, register_norm, register_position,
                       register_embedding, register_head, register_arrangement, lookup, registered)
from .base import Part, KVCacheSpec, PagedSpec, StateSpec
from . import norm, rope, attention, mlp, embedding, block  # noqa: F401  (register the built-in kinds)
from .model import DecoderModel, build_model, StepContext, KVView, StateView

__all__ = ["register_mixer", "register_feed_forward", "register_norm", "register_position",
           "register_embedding", "register_head", "register_arrangement", "lookup", "registered", "Part",
           "KVCacheSpec", "PagedSpec", "StateSpec", "DecoderModel", "build_model", "StepContext", "KVView", "StateView"]
