"""Parts a layer is put together from, and the registries that name them."""

from .attention import GroupedQueryAttention
from .base import (PAGE, Block, BorrowedCache, CompositeSpec, FeedForward, FixedStateSpec, LayerCache, Mixer, Norm, PagedKVSpec, PagedSpec,
                   PageTensor, Part, PartSpec, PositionEncoding, Runtime)
from .block import HyperConnectionBlock, OutputNormBlock, ParallelBlock, PreNormBlock
from .delta_rule import GatedDeltaRule
from .diff_attention import DifferentialAttention
from .embedding import LMHead, TokenEmbedding
from .feed_forward import ActivatedFF, PolyNormFF, SwiGLU
from .gla import GatedLinearAttention
from .hgrn2 import HGRN2
from .input_conv import ShortConvInput
from .latent_attention import LatentAttention
from .mixed_attention import MixedHeadsAttention
from .moe import RoutedExperts
from .norm import DynamicTanh, LayerNorm, RMSNorm
from .parallel_mixer import ParallelMixers
from .position import NoPosition, RotaryPosition
from .registry import build_part, part_kinds, register_part, unregister_part
from .residual import ResidualStream
from .token_input import GatedTokenInput

register_part("norm", "rmsnorm", RMSNorm)
register_part("norm", "dynamic_tanh", DynamicTanh)
register_part("norm", "layer_norm", LayerNorm)
register_part("position", "rotary", RotaryPosition)
register_part("position", "none", NoPosition)
register_part("mixer", "gqa_attention", GroupedQueryAttention)
register_part("mixer", "diff_attention", DifferentialAttention)
register_part("mixer", "gated_linear_attention", GatedLinearAttention)
register_part("mixer", "gated_delta_rule", GatedDeltaRule)
register_part("mixer", "parallel", ParallelMixers)
register_part("mixer", "latent_attention", LatentAttention)
register_part("mixer", "hgrn2", HGRN2)
register_part("mixer", "mixed_heads_attention", MixedHeadsAttention)
register_part("feed_forward", "swiglu", SwiGLU)
register_part("feed_forward", "routed_experts", RoutedExperts)
register_part("feed_forward", "poly_norm", PolyNormFF)
register_part("feed_forward", "activated", ActivatedFF)
register_part("input_conv", "short_causal", ShortConvInput)
register_part("token_input", "gated_table", GatedTokenInput)
register_part("block", "pre_norm", PreNormBlock)
register_part("block", "parallel", ParallelBlock)
register_part("block", "output_norm", OutputNormBlock)
register_part("block", "hyper_connections", HyperConnectionBlock)
register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "lm_head", LMHead)

__all__ = [
    "ActivatedFF", "Block", "BorrowedCache", "HyperConnectionBlock", "MixedHeadsAttention", "CompositeSpec", "HGRN2", "LatentAttention", "LayerNorm", "OutputNormBlock", "PolyNormFF", "ShortConvInput", "DifferentialAttention", "DynamicTanh", "GatedDeltaRule", "GatedTokenInput", "ParallelBlock", "ParallelMixers", "RoutedExperts", "FeedForward", "FixedStateSpec", "GatedLinearAttention", "GroupedQueryAttention", "LMHead", "LayerCache", "Mixer",
    "NoPosition", "Norm", "PAGE", "PageTensor", "PagedKVSpec", "PagedSpec", "Part", "PartSpec", "PositionEncoding", "PreNormBlock", "RMSNorm",
    "ResidualStream", "RotaryPosition", "Runtime", "SwiGLU", "TokenEmbedding", "build_part", "part_kinds",
    "register_part", "unregister_part",
]
