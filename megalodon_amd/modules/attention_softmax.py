"""`AttentionSoftmax` (megalodon/modules/attention_softmax.py:9-20): the
`attention_softmax` op as a module."""
import torch

from ..fused_ops import attention_softmax
from .fused_attention import _OpModule


class AttentionSoftmax(_OpModule):
    """x (..., L1, L2) -> softmax over the last axis.  With `use_causal_mask`
    row r keeps columns 0 .. L2 - L1 + r; `dropout` drops keys before the
    softmax, in training mode only."""

    def __init__(self, dropout: float = 0.0, use_causal_mask: bool = False) -> None:
        super().__init__(causal=use_causal_mask, dropout=dropout)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        o = self.options
        return attention_softmax(x, o["dropout"], o["causal"], self.training)
