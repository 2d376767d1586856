"""Typed configurations and the architecture registry."""

from .base import ConfigError, KeyReader, ModelConfig, architecture_of, read_config_json
from .engine import (DEFAULT_BLOCK_SIZE, DEFAULT_MAX_CONCURRENT, DEFAULT_NUM_BLOCKS,
                     EngineConfig, normalize_dtype)
from .gizilorn import GizilornAttention, GizilornConfig, GizilornDense, GizilornLatentAttention, GizilornLayer
from .kamedra import KamedraAttention, KamedraConfig, KamedraGLA, KamedraLayer, RotaryScaling
from .metitar import (MetitarConfig, MetitarDense, MetitarExperts, MetitarHGRN2, MetitarLatentAttention, MetitarLayer,
                      RampedScaling)
from .qwen2 import Qwen2Config
from .rusolorn import RusolornAttention, RusolornConfig, RusolornDeltaRule, RusolornExperts, RusolornLayer
from .registry import (Architecture, config_from_dict, register_architecture,
                       registered_architectures, resolve_architecture, unregister_architecture)

__all__ = [
    "Architecture", "ConfigError", "DEFAULT_BLOCK_SIZE", "DEFAULT_MAX_CONCURRENT",
    "DEFAULT_NUM_BLOCKS", "EngineConfig", "GizilornAttention", "GizilornConfig", "GizilornDense",
    "GizilornLatentAttention", "GizilornLayer", "KamedraAttention", "KamedraConfig", "KamedraGLA", "KamedraLayer", "KeyReader",
    "MetitarConfig", "MetitarDense", "MetitarExperts", "MetitarHGRN2", "MetitarLatentAttention", "MetitarLayer", "RampedScaling",
    "ModelConfig", "Qwen2Config", "RotaryScaling", "RusolornAttention", "RusolornConfig", "RusolornDeltaRule",
    "RusolornExperts", "RusolornLayer",
    "architecture_of", "config_from_dict", "normalize_dtype", "read_config_json",
    "register_architecture", "registered_architectures", "resolve_architecture",
    "unregister_architecture",
]
