"""`AttentionSoftmax` module (megalodon/modules/attention_softmax.py:9-20): the
row softmax of attention scores with optional causal mask and DropKey, as an
`nn.Module` over the `attention_softmax` op."""
import torch
import torch.nn as nn

from ..fused_ops import attention_softmax


class AttentionSoftmax(nn.Module):
    """x (..., L1, L2) -> softmax over the last axis; with `use_causal_mask` row r
    keeps columns 0 .. L2 - L1 + r; `dropout` drops keys before the softmax in
    training mode only."""

    def __init__(self, dropout: float = 0.0, use_causal_mask: bool = False) -> None:
        super().__init__()
        self._dropout = dropout
        self._use_causal_mask = use_causal_mask

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return attention_softmax(x, self._dropout, self._use_causal_mask, self.training)

    def extra_repr(self) -> str:
        # the reference formats a `_causal` attribute it never sets (:19-20)
        return f"causal={self._use_causal_mask}, dropout={self._dropout}"
