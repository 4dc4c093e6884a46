from .base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITIONS, CacheNeed, PageTensor, Part,
                   Registry, Runtime, StateNeed, TensorDecl)
from . import norm, rotary, attention, masked_attention, latent_attention, gated_delta, general_delta, matrix_memory, mixer_pair, feedforward, moe, block, embedding  # noqa: F401  (register the built-in parts)

__all__ = ["BLOCKS", "EMBEDDINGS", "FEED_FORWARDS", "HEADS", "MIXERS", "NORMS", "POSITIONS", "CacheNeed", "PageTensor",
           "Part", "Registry", "Runtime", "StateNeed", "TensorDecl"]
