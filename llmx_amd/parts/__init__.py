"""Parts a model is put together from: norms, position encodings, mixers, feed-forwards, embedding, head, blocks."""

from .base import (BuildContext, Embedding, FeedForward, Head, LayerCache, Mixer, Norm, Part, PositionEncoding, ResidualInput, build_part,
                   register, unregister)
from .spec import BlockSpec, CacheTensor, CompositeNeed, KVNeed, ModelSpec, PagedNeed, PartSpec, RunEntry, StateNeed, TensorSpec
from . import norm, position, attention, latent_attention, recurrent, linear_state, side_by_side, moe, embedding, token_input, pass_input, block  # noqa: F401  (registers the built-in parts)

__all__ = ["BuildContext", "Embedding", "FeedForward", "Head", "LayerCache", "Mixer", "Norm", "Part", "PositionEncoding", "ResidualInput",
           "build_part", "register", "unregister", "BlockSpec", "CacheTensor", "CompositeNeed", "KVNeed", "PagedNeed", "ModelSpec", "PartSpec", "RunEntry", "StateNeed",
           "TensorSpec"]
