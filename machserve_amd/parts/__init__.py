from .base import (Block, FeedForward, GroupView, Mixer, Norm, PagedKVRequest, Part, PendingNorm, PositionEncoding, ResidualStream, Runtime,
                   SharedKVRequest, StateRequest, StepContext, TensorDecl)
from .registry import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS, register_block,
                       register_embedding, register_feed_forward, register_head, register_mixer, register_norm,
                       register_position_encoding)
from . import norm, rotary, attention, feed_forward, block  # noqa: F401  (registers the built-in parts)
from .model import DecoderModel, Embedding, Head

__all__ = ["Block", "FeedForward", "GroupView", "Mixer", "Norm", "PagedKVRequest", "Part", "PendingNorm", "PositionEncoding",
           "ResidualStream", "Runtime", "SharedKVRequest", "StateRequest", "StepContext", "TensorDecl", "BLOCKS", "FEED_FORWARDS",
           "MIXERS", "NORMS", "POSITION_ENCODINGS", "EMBEDDINGS", "HEADS", "register_block", "register_feed_forward", "register_mixer",
           "register_norm", "register_position_encoding", "register_embedding", "register_head", "DecoderModel", "Embedding",
           "Head"]
