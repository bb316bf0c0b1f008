from .specs import (DiffAttentionSpec, MultiStreamLayerSpec, StateSpaceDualSpec, StreamMixSpec, ChunkedAttentionSpec, GatedRecurrenceSpec, PairEmbeddingSpec, PostNormLayerSpec, RoutedMlpSpec, SideBySideSpec, TimeMixSpec,
                    AttentionSpec, ConfigError, ConvAttentionSpec, LatentAttentionSpec, ParallelLayerSpec, EmbeddingSpec, GatedMlpSpec, HeadSpec, LayerSpec, LightningSpec, ModelSpec,
                    NormSpec, RotarySpec, SandwichLayerSpec, SelectiveScanSpec, TalkingAttentionSpec, YarnSpec)
from .registry import architectures, architecture_of, config_from_dict, load_config, register_architecture
from .qwen2 import ARCHITECTURE as QWEN2_ARCHITECTURE, Qwen2Config
from .renanex import ARCHITECTURE as RENANEX_ARCHITECTURE, RenanexConfig
from .nubodra import ARCHITECTURE as NUBODRA_ARCHITECTURE, NubodraConfig
from .melerax import ARCHITECTURE as MELERAX_ARCHITECTURE, MeleraxConfig
from .befirax import ARCHITECTURE as BEFIRAX_ARCHITECTURE, BefiraxConfig

register_architecture(QWEN2_ARCHITECTURE, Qwen2Config, model_type="qwen2")
register_architecture(RENANEX_ARCHITECTURE, RenanexConfig)
register_architecture(NUBODRA_ARCHITECTURE, NubodraConfig)
register_architecture(MELERAX_ARCHITECTURE, MeleraxConfig)
register_architecture(BEFIRAX_ARCHITECTURE, BefiraxConfig)

__all__ = ["BefiraxConfig", "BEFIRAX_ARCHITECTURE", "DiffAttentionSpec", "MultiStreamLayerSpec", "StateSpaceDualSpec", "StreamMixSpec", "ChunkedAttentionSpec", "GatedRecurrenceSpec", "PairEmbeddingSpec", "PostNormLayerSpec", "RoutedMlpSpec", "SideBySideSpec", "TimeMixSpec",
           "MeleraxConfig", "MELERAX_ARCHITECTURE", "AttentionSpec", "ConfigError", "ConvAttentionSpec", "LatentAttentionSpec", "ParallelLayerSpec", "NubodraConfig", "NUBODRA_ARCHITECTURE", "EmbeddingSpec", "GatedMlpSpec", "HeadSpec", "LayerSpec", "LightningSpec", "ModelSpec",
           "NormSpec", "RotarySpec", "SandwichLayerSpec", "SelectiveScanSpec", "TalkingAttentionSpec", "YarnSpec", "architectures", "architecture_of", "config_from_dict", "load_config",
           "register_architecture", "Qwen2Config", "QWEN2_ARCHITECTURE", "RenanexConfig", "RENANEX_ARCHITECTURE"]
