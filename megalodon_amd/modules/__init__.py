"""Modules with the reference's names (megalodon/modules/__init__.py:1-15) for the hot path."""
from .attention_softmax import AttentionSoftmax
from .chunk_attention import _InnerAttention, apply_rotary_emb
from .complex_exponential_moving_average import MultiHeadComplexEMA
from .fused_attention import SwiftAttention
from .layer_norm import FusedLayerNorm, FusedRMSNorm
from .moving_average_gated_attention import MegaBlock, MovingAverageGatedAttention
from .normalized_feedforward_network import NormalizedFeedForwardNetwork
from .rotary_positional_embedding import RotaryEmbedding
from .timestep_norm import TimestepNorm, TimestepNormFunc, timestep_norm

__all__ = ["MegaBlock", "MovingAverageGatedAttention", "NormalizedFeedForwardNetwork", "FusedLayerNorm",
           "FusedRMSNorm", "MultiHeadComplexEMA", "TimestepNorm", "TimestepNormFunc", "timestep_norm", "_InnerAttention",
           "apply_rotary_emb", "RotaryEmbedding", "AttentionSoftmax", "SwiftAttention"]
