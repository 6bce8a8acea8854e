"""`nn.Linear` whose input gradient is computed from a transposed copy of the weight.

With model-parallel world size 1 the reference's Column/RowParallelLinear are
`F.linear` (megalodon/modules/model_parallel/layers.py:222-235,321-341), whose
backward forms `dx = dy @ W` with W (out, in) read along its rows.  On MI355X
the library GEMM is 13-24 % faster when both operands run along the reduction
axis (`dy @ Wt^T` with Wt = W^T contiguous, the same layout the forward
`x @ W^T` uses), and the tiled transpose of W costs 15-30 us, so the backward
makes that copy.  Values are those of `F.linear`; parameters keep the names
and shapes of `nn.Linear`, so state dicts are interchangeable."""
from typing import Optional, Tuple

import torch
import torch.nn.functional as F
from torch import nn
from torch.autograd.function import FunctionCtx

from .. import extension as megalodon_ops


class LinearFunc(torch.autograd.Function):
    """y = x W^T (+ bias) (+ residual).  A residual goes into the GEMM as its
    accumulator input (`addmm`, one pass fewer over the activation than a
    separate add); it needs a layer without bias."""

    @staticmethod
    def forward(ctx: FunctionCtx, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                residual: Optional[torch.Tensor]) -> torch.Tensor:
        ctx.save_for_backward(x, weight)
        ctx.has_bias = bias is not None
        ctx.has_residual = residual is not None
        if residual is None:
            return F.linear(x, weight, bias)
        out_shape = x.shape[:-1] + (weight.shape[0],)
        y = torch.addmm(residual.reshape(-1, weight.shape[0]), x.reshape(-1, x.shape[-1]), weight.t())
        return y.view(out_shape)

    @staticmethod
    def backward(ctx: FunctionCtx, y_grad: torch.Tensor) -> Tuple[Optional[torch.Tensor], ...]:
        x, weight = ctx.saved_tensors
        g2 = y_grad.reshape(-1, y_grad.shape[-1])
        dx = dw = db = None
        if ctx.needs_input_grad[0]:
            wt = megalodon_ops.transpose_last2(weight)          # (in, out), rows along the reduction axis
            dx = F.linear(g2, wt).view(x.shape)
        if ctx.needs_input_grad[1]:
            dw = g2.t() @ x.reshape(-1, x.shape[-1])
        if ctx.has_bias and ctx.needs_input_grad[2]:
            db = g2.sum(0)
        return dx, dw, db, (y_grad if ctx.has_residual and ctx.needs_input_grad[3] else None)


class Linear(nn.Linear):
    """Drop-in for `nn.Linear` (same parameters, same values); `residual`, for
    layers without bias, is added inside the GEMM."""

    def forward(self, x: torch.Tensor, residual: Optional[torch.Tensor] = None) -> torch.Tensor:
        fused = (x.is_cuda and x.dtype in (torch.bfloat16, torch.float16) and self.weight.dtype == x.dtype)
        if residual is not None and (self.bias is not None or not fused or residual.dtype != x.dtype):
            return F.linear(x, self.weight, self.bias) + residual
        if fused and torch.is_grad_enabled() and (x.requires_grad or self.weight.requires_grad
                                                  or (residual is not None and residual.requires_grad)):
            return LinearFunc.apply(x, self.weight, self.bias, residual)
        if residual is not None:
            return torch.addmm(residual.reshape(-1, self.weight.shape[0]), x.reshape(-1, x.shape[-1]),
                               self.weight.t()).view(x.shape[:-1] + (self.weight.shape[0],))
        return F.linear(x, self.weight, self.bias)
