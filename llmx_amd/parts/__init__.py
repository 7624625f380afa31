"""Parts a model is put together from: norms, position encodings, mixers, feed-forwards, embedding, head, blocks."""

from .base import (BuildContext, Embedding, FeedForward, Head, LayerCache, Mixer, Norm, Part, PositionEncoding, build_part,
                   register, unregister)
from .spec import BlockSpec, CacheTensor, KVNeed, ModelSpec, PagedNeed, PartSpec, RunEntry, StateNeed, TensorSpec
from . import norm, position, attention, moe, embedding, block  # noqa: F401  (registers the built-in parts)

__all__ = ["BuildContext", "Embedding", "FeedForward", "Head", "LayerCache", "Mixer", "Norm", "Part", "PositionEncoding",
           "build_part", "register", "unregister", "BlockSpec", "CacheTensor", "KVNeed", "PagedNeed", "ModelSpec", "PartSpec", "RunEntry", "StateNeed",
           "TensorSpec"]
