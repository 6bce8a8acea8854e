"""Fused attention `softmax(scale q k^T) v` on (B, L, N, H) tensors, under the
names of megalodon/modules/fused_ops/attention/swift.py:9-95:

* `swift_efficient_attention(q, k, v, scale, dropout, use_causal_mask, training)`
  -- differentiable; keeps (q, k, v, P) for the backward pass,
* `swift_efficient_attention_fwd/bwd` -- the two halves for callers that run
  their own backward (the reference's chunk-parallel code does)."""
from typing import Optional, Tuple

import torch

from ... import extension as ops
from .._autograd import fused_op


def _rate(dropout: float, training: bool) -> float:
    return dropout if training else 0.0  # DropKey acts in training mode only


def _run(q, k, v, scale=1.0, dropout=0.0, use_causal_mask=True, training=True):
    # w goes to the backward pass and nowhere else: the zeros right of the diagonal block stay unwritten
    y, w = ops.attention_fwd(q, k, v, scale, _rate(dropout, training), use_causal_mask, lower_only=True)
    return y, (q, k, v, w), (scale, use_causal_mask)


def _grad(consts, saved, y_grad):
    scale, causal = consts
    return (*ops.attention_bwd(y_grad, *saved, scale, causal), None, None, None, None)


FusedAttentionFunc = fused_op("FusedAttentionFunc", _run, _grad, doc=__doc__)
swift_efficient_attention = FusedAttentionFunc.apply


def swift_efficient_attention_fwd(q, k, v, scale: float = 1.0, dropout: float = 0.0, use_causal_mask: bool = True,
                                  training: bool = True,
                                  requires_grad: bool = False) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """(y, P); P is handed back only when a backward call will follow."""
    if requires_grad and not training:
        raise AssertionError("requires_grad needs training mode")
    y, w = ops.attention_fwd(q, k, v, scale, _rate(dropout, training), use_causal_mask)
    return y, (w if requires_grad else None)


def swift_efficient_attention_bwd(grad, q, k, v, w, scale: float = 1.0, use_causal_mask: bool = True):
    """(dq, dk, dv) from the P that `swift_efficient_attention_fwd` returned."""
    return ops.attention_bwd(grad, q, k, v, w, scale, use_causal_mask)
