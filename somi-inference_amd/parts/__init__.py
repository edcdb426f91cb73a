"""Parts a layer is put together from, and the registries that name them."""

from .attention import GroupedQueryAttention
from .base import (PAGE, Block, CompositeSpec, FeedForward, FixedStateSpec, LayerCache, Mixer, Norm, PagedKVSpec, PagedSpec,
                   PageTensor, Part, PartSpec, PositionEncoding, Runtime)
from .block import ParallelBlock, PreNormBlock
from .delta_rule import GatedDeltaRule
from .diff_attention import DifferentialAttention
from .embedding import LMHead, TokenEmbedding
from .feed_forward import SwiGLU
from .gla import GatedLinearAttention
from .moe import RoutedExperts
from .norm import DynamicTanh, RMSNorm
from .parallel_mixer import ParallelMixers
from .position import NoPosition, RotaryPosition
from .registry import build_part, part_kinds, register_part, unregister_part
from .residual import ResidualStream
from .token_input import GatedTokenInput

register_part("norm", "rmsnorm", RMSNorm)
register_part("norm", "dynamic_tanh", DynamicTanh)
register_part("position", "rotary", RotaryPosition)
register_part("position", "none", NoPosition)
register_part("mixer", "gqa_attention", GroupedQueryAttention)
register_part("mixer", "diff_attention", DifferentialAttention)
register_part("mixer", "gated_linear_attention", GatedLinearAttention)
register_part("mixer", "gated_delta_rule", GatedDeltaRule)
register_part("mixer", "parallel", ParallelMixers)
register_part("feed_forward", "swiglu", SwiGLU)
register_part("feed_forward", "routed_experts", RoutedExperts)
register_part("token_input", "gated_table", GatedTokenInput)
register_part("block", "pre_norm", PreNormBlock)
register_part("block", "parallel", ParallelBlock)
register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "lm_head", LMHead)

__all__ = [
    "Block", "CompositeSpec", "DifferentialAttention", "DynamicTanh", "GatedDeltaRule", "GatedTokenInput", "ParallelBlock", "ParallelMixers", "RoutedExperts", "FeedForward", "FixedStateSpec", "GatedLinearAttention", "GroupedQueryAttention", "LMHead", "LayerCache", "Mixer",
    "NoPosition", "Norm", "PAGE", "PageTensor", "PagedKVSpec", "PagedSpec", "Part", "PartSpec", "PositionEncoding", "PreNormBlock", "RMSNorm",
    "ResidualStream", "RotaryPosition", "Runtime", "SwiGLU", "TokenEmbedding", "build_part", "part_kinds",
    "register_part", "unregister_part",
]
