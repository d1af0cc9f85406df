from .base import (AttentionSpec, BlockSpec, CappedAttentionSpec, ConfigError, DenseFFSpec, GatedDeltaSpec, HyperBlockSpec, LatentAttentionSpec,
                   LayerNormSpec, MLSTMSpec, ModelConfig, ModelSpec, PairRotarySpec, ParallelMixerSpec, PartSpec, PostNormBlockSpec, RMSNormSpec,
                   RotarySpec, RoutedExpertsSpec, RunEntry, SwiGLUSpec)
from .migurax import MiguraxConfig
from .nebutar import NebutarConfig
from .qwen2 import Qwen2Config

__all__ = ["AttentionSpec", "BlockSpec", "CappedAttentionSpec", "ConfigError", "DenseFFSpec", "GatedDeltaSpec", "HyperBlockSpec",
           "LatentAttentionSpec", "LayerNormSpec", "MLSTMSpec", "ModelConfig", "ModelSpec", "PairRotarySpec", "ParallelMixerSpec", "PartSpec",
           "PostNormBlockSpec", "RMSNormSpec", "RotarySpec", "RoutedExpertsSpec", "RunEntry", "SwiGLUSpec", "MiguraxConfig", "NebutarConfig",
           "Qwen2Config"]
