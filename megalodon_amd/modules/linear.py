"""`nn.Linear` whose input gradient is computed from a transposed copy of the weight.

With model-parallel world size 1 the reference's Column/RowParallelLinear are
`F.linear` (megalodon/modules/model_parallel/layers.py:222-235,321-341), whose
backward forms `dx = dy @ W` with W (out, in) read along its rows.  On MI355X
the library GEMM is 13-24 % faster when both operands run along the reduction
axis (`dy @ Wt^T` with Wt = W^T contiguous, the same layout the forward
`x @ W^T` uses), and the tiled transpose of W costs 15-30 us, so the backward
makes that copy; the weight gradient of the large layers runs on the attention
operator's product kernel (`_weight_grad`).  Values are those of `F.linear`;
parameters keep the names and shapes of `nn.Linear`, so state dicts are
interchangeable."""
from typing import Optional, Tuple

import torch
import torch.nn.functional as F
from torch import nn
from torch.autograd.function import FunctionCtx

from .. import extension as megalodon_ops


def _weight_grad(g2: torch.Tensor, x2: torch.Tensor) -> torch.Tensor:
    """dW = g2^T x2, (out, in) from (tokens, out) and (tokens, in).  Both operands run across
    the reduction axis (tokens) here, the slowest layout of the library GEMM on MI355X
    (0.9-1.2 PFLOP/s at 32768 tokens against 1.5 for the forward's layout).  The attention
    operator's product kernel takes exactly this layout (dV = P^T dY) and measured, at 32768
    tokens, out x in = 11008 x 4096: 2.16 ms against 3.28 (3.16 with one operand transposed
    first), 4096 x 11008: 2.22 / 3.13, 8192 x 4096: 1.54 / 1.87, 4096 x 4096: 0.78 / 0.92;
    below one 256 x 256 tile per compute unit (1024 x 4096: 0.50 / 0.28 ms) the library stays."""
    n_out, n_in = g2.shape[1], x2.shape[1]
    tiles = ((n_out + 255) // 256) * ((n_in + 255) // 256)
    # (operands of 2^30 elements and more leave the kernel's aligned path, whose offsets are 32-bit)
    if (g2.dtype in (torch.bfloat16, torch.float16) and g2.shape[0] >= 4096 and g2.shape[0] % 32 == 0
            and n_out % 8 == 0 and n_in % 8 == 0 and tiles >= 256
            and g2.shape[0] * max(n_out, n_in) < (1 << 30)):
        return megalodon_ops.linear_weight_grad(g2, x2)
    return g2.t() @ x2


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
            dw = _weight_grad(g2, x.reshape(-1, x.shape[-1]))
        if ctx.has_bias and ctx.needs_input_grad[2]:
            db = g2.sum(0)
        return dx, dw, db, (y_grad if ctx.has_residual and ctx.needs_input_grad[3] else None)


class LinearGroupFunc(torch.autograd.Function):
    """Several bias-optional linear layers of one input: (y_1, ..., y_n) = (x W_1^T + b_1, ...).
    The forward is n separate products; the backward forms the input gradient as one
    accumulation -- dx = dy_1 W_1, then dx += dy_i W_i inside the GEMM (`addmm_`) -- instead of n
    gradients that autograd adds up with n - 1 passes over the activation."""

    @staticmethod
    def forward(ctx: FunctionCtx, x: torch.Tensor, *params: Optional[torch.Tensor]):
        weights, biases = params[0::2], params[1::2]
        ctx.save_for_backward(x, *weights)
        ctx.has_bias = [b is not None for b in biases]
        return tuple(F.linear(x, w, b) for w, b in zip(weights, biases))

    @staticmethod
    def backward(ctx: FunctionCtx, *y_grads: torch.Tensor):
        x, *weights = ctx.saved_tensors
        x2 = x.reshape(-1, x.shape[-1])
        dx = None
        grads = []
        for i, (w, g) in enumerate(zip(weights, y_grads)):
            g2 = g.reshape(-1, g.shape[-1])
            if ctx.needs_input_grad[0]:
                wt = megalodon_ops.transpose_last2(w)      # (in, out), rows along the reduction axis
                if dx is None:
                    dx = F.linear(g2, wt)
                else:
                    dx.addmm_(g2, wt.t())
            dw = _weight_grad(g2, x2) if ctx.needs_input_grad[1 + 2 * i] else None
            db = g2.sum(0) if ctx.has_bias[i] and ctx.needs_input_grad[2 + 2 * i] else None
            grads += [dw, db]
        return (None if dx is None else dx.view(x.shape), *grads)


def linear_group(x: torch.Tensor, layers) -> Tuple[torch.Tensor, ...]:
    """`tuple(layer(x) for layer in layers)` for `Linear` layers that read the same input; on the
    GPU in 16 bits with gradients enabled their backward shares one input-gradient accumulation."""
    layers = list(layers)
    fused = (x.is_cuda and x.dtype in (torch.bfloat16, torch.float16) and torch.is_grad_enabled()
             and all(l.weight.dtype == x.dtype for l in layers)
             and (x.requires_grad or any(l.weight.requires_grad for l in layers)))
    if not fused or len(layers) < 2:
        return tuple(l(x) for l in layers)
    params = []
    for l in layers:
        params += [l.weight, l.bias]
    return LinearGroupFunc.apply(x, *params)


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
