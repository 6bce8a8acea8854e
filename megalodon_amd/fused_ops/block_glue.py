"""Autograd wrappers of the block's memory-bound glue kernels.

The reference writes these steps as plain PyTorch expressions
(megalodon/modules/moving_average_gated_attention.py:299-300,314,333-336,
megalodon/modules/normalized_feedforward_network.py:82); here each is one
streaming kernel forward and one backward."""
from typing import Optional, Tuple

import torch
from torch.autograd.function import FunctionCtx

from .. import extension as megalodon_ops


class TransposeLast2Func(torch.autograd.Function):
    """`x.transpose(-2, -1).contiguous()`; the gradient is the same move back."""

    @staticmethod
    def forward(ctx: FunctionCtx, x: torch.Tensor) -> torch.Tensor:
        return megalodon_ops.transpose_last2(x)

    @staticmethod
    def backward(ctx: FunctionCtx, y_grad: torch.Tensor) -> torch.Tensor:
        return megalodon_ops.transpose_last2(y_grad)


class SiluMulFunc(torch.autograd.Function):
    """`F.silu(a) * b` saving only (a, b)."""

    @staticmethod
    def forward(ctx: FunctionCtx, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
        ctx.save_for_backward(a, b)
        return megalodon_ops.silu_mul_fwd(a, b)

    @staticmethod
    def backward(ctx: FunctionCtx, out_grad: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        a, b = ctx.saved_tensors
        return megalodon_ops.silu_mul_bwd(out_grad, a, b)


class LayerNormPlusOneFunc(torch.autograd.Function):
    """LayerNorm / RMSNorm whose stored weight is gamma - 1
    (megalodon/modules/layer_norm.py:30-33,62-65); saves x and the row statistics."""

    @staticmethod
    def forward(ctx: FunctionCtx, x: torch.Tensor, weight: Optional[torch.Tensor], bias: Optional[torch.Tensor],
                eps: float, rms: bool) -> torch.Tensor:
        y, mean, rstd = megalodon_ops.layer_norm_fwd(x, weight, bias, eps, rms)
        ctx.save_for_backward(x, weight, mean, rstd)
        ctx.rms = rms
        ctx.has_bias = bias is not None
        return y

    @staticmethod
    def backward(ctx: FunctionCtx, y_grad: torch.Tensor):
        x, weight, mean, rstd = ctx.saved_tensors
        dx, dw, db = megalodon_ops.layer_norm_bwd(y_grad, x, weight, mean, rstd, ctx.rms, ctx.has_bias)
        return dx, dw, db, None, None


class QkNormRotaryFunc(torch.autograd.Function):
    """z -> (q, k) in one pass (moving_average_gated_attention.py:319-330 plus the
    rotary product of rotary_positional_embedding.py:53-77)."""

    @staticmethod
    def forward(ctx: FunctionCtx, z: torch.Tensor, gamma: torch.Tensor, beta: torch.Tensor,
                freqs_cis: Optional[torch.Tensor], head_dim: int, eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
        q, k, rstd = megalodon_ops.qk_norm_rotary_fwd(z, gamma, beta, freqs_cis, head_dim, eps)
        ctx.save_for_backward(z, gamma, rstd)
        ctx.freqs_cis = freqs_cis
        ctx.head_dim = head_dim
        return q, k

    @staticmethod
    def backward(ctx: FunctionCtx, q_grad: torch.Tensor, k_grad: torch.Tensor):
        z, gamma, rstd = ctx.saved_tensors
        dz, dgamma, dbeta = megalodon_ops.qk_norm_rotary_bwd(q_grad, k_grad, z, gamma, rstd, ctx.freqs_cis,
                                                             ctx.head_dim)
        return dz, dgamma, dbeta, None, None, None


qk_norm_rotary = QkNormRotaryFunc.apply


def layer_norm_plus_one(x: torch.Tensor, weight: Optional[torch.Tensor], bias: Optional[torch.Tensor],
                        eps: float = 1e-5, rms: bool = False) -> torch.Tensor:
    return LayerNormPlusOneFunc.apply(x, weight, bias, eps, rms)


transpose_last2 = TransposeLast2Func.apply
silu_mul = SiluMulFunc.apply
