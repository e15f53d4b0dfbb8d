from .model_config import (ChannelDeltaConfig, ChunkAttentionConfig, ConfigError, ExpertsConfig, GatedAttentionConfig,
                           KirisunConfig, KirisunLayer, MafaraxConfig, MafaraxLayer, NozuraxConfig, NozuraxLayer, Qwen3Config,
                           SoftmaxExpertsConfig, StateSpaceConfig, canonical_dtype, read_config_json, PemuvikConfig, PemuvikLayer,
                           SigmoidAttentionConfig, LatentAttentionConfig, ChoiceExpertsConfig)
from .engine_config import EngineConfig
from .registry import (Architecture, register_architecture, get_architecture,
                       architecture_of, known_architectures)

__all__ = ["ConfigError", "Qwen3Config", "NozuraxConfig", "NozuraxLayer", "MafaraxConfig", "MafaraxLayer",
           "ChunkAttentionConfig", "StateSpaceConfig", "ExpertsConfig", "KirisunConfig", "KirisunLayer", "GatedAttentionConfig",
           "ChannelDeltaConfig", "SoftmaxExpertsConfig", "PemuvikConfig", "PemuvikLayer", "SigmoidAttentionConfig",
           "LatentAttentionConfig", "ChoiceExpertsConfig", "canonical_dtype", "read_config_json", "EngineConfig",
           "Architecture", "register_architecture", "get_architecture", "architecture_of",
           "known_architectures"]
