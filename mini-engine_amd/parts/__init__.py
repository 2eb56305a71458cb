"""Parts of a decoder layer. Importing this package registers the built-in kinds."""

from . import attention, decay_state, delta_rule, latent_attention, mlp, norm, pair, rotary, routed_experts, time_mix  # noqa: F401
from .base import (
    BLOCK_ARRANGEMENTS,
    FEED_FORWARDS,
    MIXERS,
    NORMS,
    POSITION_ENCODINGS,
    FeedForward,
    KVBinding,
    KVCacheNeed,
    Mixer,
    Norm,
    PairBinding,
    PositionEncoding,
    StateBinding,
    StateNeed,
)
from .block import HyperConnectionBlock, ParallelBlock, PreNormBlock, ResultNormBlock, build_block
from .decoder import Decoder

__all__ = [
    "BLOCK_ARRANGEMENTS",
    "Decoder",
    "FEED_FORWARDS",
    "FeedForward",
    "HyperConnectionBlock",
    "KVBinding",
    "KVCacheNeed",
    "MIXERS",
    "Mixer",
    "NORMS",
    "Norm",
    "PairBinding",
    "POSITION_ENCODINGS",
    "ParallelBlock",
    "PositionEncoding",
    "PreNormBlock",
    "StateBinding",
    "StateNeed",
    "build_block",
]
