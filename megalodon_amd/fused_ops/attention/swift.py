"""Fused attention autograd op (mirror of
megalodon/modules/fused_ops/attention/swift.py:9-95)."""
from typing import Optional, Tuple

import torch
from torch.autograd.function import FunctionCtx

from ... import extension as megalodon_ops


class FusedAttentionFunc(torch.autograd.Function):

    @staticmethod
    def forward(
        ctx: FunctionCtx,
        q: torch.Tensor,
        k: torch.Tensor,
        v: torch.Tensor,
        scale: float = 1.0,
        dropout: float = 0.0,
        use_causal_mask: bool = True,
        training: bool = True,
    ) -> torch.Tensor:
        p = dropout if training else 0.0
        y, w = _fused_efficient_attention_fwd(q, k, v, scale, p, use_causal_mask)
        ctx.save_for_backward(q, k, v, w)
        ctx.scale = scale
        ctx.use_causal_mask = use_causal_mask
        return y

    @staticmethod
    def backward(ctx: FunctionCtx, y_grad: torch.Tensor):
        q, k, v, w = ctx.saved_tensors
        q_grad, k_grad, v_grad = _fused_efficient_attention_bwd(y_grad, q, k, v, w, ctx.scale, ctx.use_causal_mask)
        return q_grad, k_grad, v_grad, None, None, None, None


def _fused_efficient_attention_fwd(q, k, v, scale: float = 1.0, dropout: float = 0.0,
                                   use_causal_mask: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
    return megalodon_ops.attention_fwd(q, k, v, scale, dropout, use_causal_mask)


def _fused_efficient_attention_bwd(grad, q, k, v, w, scale: float = 1.0, use_causal_mask: bool = True):
    return megalodon_ops.attention_bwd(grad, q, k, v, w, scale, use_causal_mask)


swift_efficient_attention = FusedAttentionFunc.apply


def swift_efficient_attention_fwd(q, k, v, scale: float = 1.0, dropout: float = 0.0,
                                  use_causal_mask: bool = True, training: bool = True,
                                  requires_grad: bool = False) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    assert training or not requires_grad
    p = dropout if training else 0.0
    y, w = _fused_efficient_attention_fwd(q, k, v, scale, p, use_causal_mask)
    w = w if requires_grad else None
    return y, w


def swift_efficient_attention_bwd(grad, q, k, v, w, scale: float = 1.0, use_causal_mask: bool = True):
    return _fused_efficient_attention_bwd(grad, q, k, v, w, scale, use_causal_mask)
