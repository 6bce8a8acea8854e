"""`SwiftAttention` module (megalodon/modules/fused_attention.py:7-20):
softmax(scale q k^T) v on (B, L, N, H) tensors as an `nn.Module` over the fused
attention op."""
import torch
import torch.nn as nn

from ..fused_ops import swift_efficient_attention


class SwiftAttention(nn.Module):
    """q, k (B, L, N, H1), v (B, L, N, H2) -> (B, L, N, H2); DropKey with rate
    `dropout` in training mode only."""

    def __init__(self, scale: float = 1.0, dropout: float = 0.0, use_causal_mask: bool = True) -> None:
        super().__init__()
        self._scale = scale
        self._dropout = dropout
        self._use_causal_mask = use_causal_mask

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        return swift_efficient_attention(q, k, v, self._scale, self._dropout, self._use_causal_mask, self.training)

    def extra_repr(self) -> str:
        return f"causal={self._use_causal_mask}, scale={self._scale}, dropout={self._dropout}"
