"""`SwiftAttention` (megalodon/modules/fused_attention.py:7-20): the fused
attention op as a module, and the small base it shares with `AttentionSoftmax`."""
import torch
import torch.nn as nn

from ..fused_ops import swift_efficient_attention


class _OpModule(nn.Module):
    """A parameter-free module around one fused op: keeps the op's options and
    prints them.  (The reference's two modules format a `_causal` attribute
    that their constructors never set.)"""

    def __init__(self, **options) -> None:
        super().__init__()
        self.options = options

    def extra_repr(self) -> str:
        return ", ".join(f"{k}={v}" for k, v in self.options.items())


class SwiftAttention(_OpModule):
    """q, k (B, L, N, H1), v (B, L, N, H2) -> softmax(scale q k^T) v of shape
    (B, L, N, H2); DropKey with rate `dropout` in training mode only."""

    def __init__(self, scale: float = 1.0, dropout: float = 0.0, use_causal_mask: bool = True) -> None:
        super().__init__(causal=use_causal_mask, scale=scale, dropout=dropout)

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        o = self.options
        return swift_efficient_attention(q, k, v, o["scale"], o["dropout"], o["causal"], self.training)
