from .base import (ARRANGEMENTS, CONNECTIONS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS, FeedForward,
                   FixedState, Mixer, Norm, NormEmit, NormedInput, PagedKV, PagedKeysValues, Part, PositionEncoding, Runtime, as_normed,
                   build_part, need_kind)
from .spec import BlockSpec, ModelSpec, ParamSpec, PartSpec, PlanEntry
from . import attention, block, connection, conv_attention, embedding, linear_attention, mlp, norm, parallel, rope, routed, selective_scan, sink_attention  # noqa: F401  (registers the built-in parts)
from .block import Block

__all__ = ["ARRANGEMENTS", "CONNECTIONS", "EMBEDDINGS", "FEED_FORWARDS", "HEADS", "MIXERS", "NORMS", "POSITION_ENCODINGS",
           "FeedForward", "FixedState", "Mixer", "Norm", "PagedKV", "PagedKeysValues", "Part", "PositionEncoding", "Runtime",
           "build_part", "need_kind", "NormEmit", "NormedInput", "as_normed", "BlockSpec", "ModelSpec", "ParamSpec", "PartSpec", "PlanEntry", "Block"]
