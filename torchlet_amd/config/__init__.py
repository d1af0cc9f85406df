from .base import (AttentionSpec, BlockSpec, ConfigError, DenseFFSpec, LatentAttentionSpec, MLSTMSpec, ModelConfig, ModelSpec,
                   PairRotarySpec, PartSpec, PostNormBlockSpec, RMSNormSpec, RotarySpec, RoutedExpertsSpec, RunEntry, SwiGLUSpec)
from .migurax import MiguraxConfig
from .qwen2 import Qwen2Config

__all__ = ["AttentionSpec", "BlockSpec", "ConfigError", "DenseFFSpec", "LatentAttentionSpec", "MLSTMSpec", "ModelConfig", "ModelSpec",
           "PairRotarySpec", "PartSpec", "PostNormBlockSpec", "RMSNormSpec", "RotarySpec", "RoutedExpertsSpec", "RunEntry",
           "SwiGLUSpec", "MiguraxConfig", "Qwen2Config"]
