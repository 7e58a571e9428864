from .base import (Part, Norm, PositionEncoding, QKTransform, Mixer, FeedForward, Block, ParamSpec, KVSpec, StateSpec,
                   RotaryParams, Runtime, make_part, make_block, unregister, register_norm, register_position,
                   register_qk_transform, register_mixer, register_feed_forward, register_block, register_embedding, register_head,
                   register_filter, SequenceFilter, register_connection, Connection, register_injection, Injection)
from . import norm, rotary, embedding, head, mlp, attention, block, filters, pooled_attention, recurrent, latent_attention    # noqa: F401  (registers the built-in parts)
from . import qk_norm, injection, parallel    # noqa: F401
from .norm import RMSNorm, LayerNorm, DynamicTanh
from .qk_norm import HeadRMSNorm
from .injection import ConcatProjection, StepAddition
from .parallel import ParallelMixers
from .filters import CausalConv
from .pooled_attention import PooledWindowAttention
from .recurrent import Retention, GatedDelta, TimeMixWKV, GatedLinearAttention
from .rotary import Rotary, NoPosition, rotary_inv_freq
from .embedding import TokenEmbedding, PairHashEmbedding
from .head import LinearHead
from .mlp import GatedMLP, DenseMLP, RoutedExperts
from .latent_attention import LatentAttention
from .attention import PagedAttention
from .block import PreNormBlock, FilteredPreNormBlock, StreamsPreNormBlock, StreamConnection, SandwichBlock

__all__ = [
    "Part", "Norm", "PositionEncoding", "QKTransform", "Mixer", "FeedForward", "Block", "ParamSpec", "KVSpec", "StateSpec",
    "RotaryParams", "Runtime", "make_part", "make_block", "unregister", "register_norm", "register_position",
    "register_qk_transform", "register_mixer", "register_feed_forward", "register_block", "register_embedding", "register_head",
    "RMSNorm", "Rotary", "NoPosition", "rotary_inv_freq", "TokenEmbedding", "LinearHead", "GatedMLP",
    "PagedAttention", "PreNormBlock", "register_filter", "SequenceFilter", "LayerNorm", "CausalConv", "PooledWindowAttention",
    "Retention", "GatedDelta", "DenseMLP", "FilteredPreNormBlock", "register_connection", "Connection", "PairHashEmbedding",
    "RoutedExperts", "LatentAttention", "StreamsPreNormBlock", "StreamConnection", "DynamicTanh", "HeadRMSNorm",
    "ConcatProjection", "TimeMixWKV", "SandwichBlock", "register_injection", "Injection", "StepAddition", "ParallelMixers",
    "GatedLinearAttention",
]
