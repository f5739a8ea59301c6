from .base import (AttentionSpec, BlockSpec, CappedAttentionSpec, ConfigError, DecayedLinearSpec, DenseFFSpec, GatedDeltaSpec, HalfRotarySpec,
                   HashedBigramSpec, HyperBlockSpec, LatentAttentionSpec, SandwichBlockSpec, ScalarRMSNormSpec,
                   LayerNormSpec, MLSTMSpec, ModelConfig, ModelSpec, PairRotarySpec, ParallelMixerSpec, PartSpec, PostNormBlockSpec, RMSNormSpec,
                   RotarySpec, RoutedExpertsSpec, RunEntry, SwiGLUSpec, OffsetRMSNormSpec, SelectiveStateSpec)
from .bafulorn import BafulornConfig
from .fotovik import FotovikConfig
from .migurax import MiguraxConfig
from .nebutar import NebutarConfig
from .qwen2 import Qwen2Config

__all__ = ["DecayedLinearSpec", "HalfRotarySpec", "HashedBigramSpec", "SandwichBlockSpec", "ScalarRMSNormSpec", "AttentionSpec", "BlockSpec", "CappedAttentionSpec", "ConfigError", "DenseFFSpec", "GatedDeltaSpec", "HyperBlockSpec",
           "LatentAttentionSpec", "LayerNormSpec", "MLSTMSpec", "ModelConfig", "ModelSpec", "PairRotarySpec", "ParallelMixerSpec", "PartSpec",
           "PostNormBlockSpec", "RMSNormSpec", "RotarySpec", "RoutedExpertsSpec", "RunEntry", "SwiGLUSpec", "FotovikConfig", "MiguraxConfig", "NebutarConfig",
           "Qwen2Config", "OffsetRMSNormSpec", "SelectiveStateSpec", "BafulornConfig"]
