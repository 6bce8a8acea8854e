"""Dropout that keeps neither the mask nor a copy of the generator (mirror of
megalodon/modules/fused_ops/memory_efficient_dropout.py:8-96).

The reference saves the CUDA generator's state in the forward and replays the
generator in the backward.  Here `rng_state` is the pair (seed, offset) taken
from the device generator, and the kernel derives the mask from it and the
element index alone, so the backward is the same launch on the gradient."""
from typing import Optional, Tuple

import torch
from torch.autograd.function import FunctionCtx

from .. import extension as megalodon_ops


class MemoryEfficientDropoutFunc(torch.autograd.Function):

    @staticmethod
    def forward(ctx: FunctionCtx, x: torch.Tensor, p: float = 0.0, training: bool = True) -> torch.Tensor:
        y, rng_state = memory_efficient_dropout_fwd(x, p, training)
        ctx.rng_state = rng_state
        ctx.p = p
        return y

    @staticmethod
    def backward(ctx: FunctionCtx, y_grad: torch.Tensor) -> Tuple[torch.Tensor, None, None]:
        return memory_efficient_dropout_bwd(y_grad, ctx.p, ctx.rng_state), None, None


def memory_efficient_dropout(x: torch.Tensor, p: float = 0.0, training: bool = True) -> torch.Tensor:
    """The reference binds this name to `MemoryEfficientDropoutFunc.apply` (:36);
    the identity cases return `x` itself so that they add no autograd node."""
    if 0.0 <= p <= 1.0 and (not training or p == 0):
        return x
    return MemoryEfficientDropoutFunc.apply(x, p, training)


def memory_efficient_dropout_fwd(x: torch.Tensor, p: float, training: bool,
                                 rng_state: Optional[Tuple[int, int]] = None
                                 ) -> Tuple[torch.Tensor, Optional[Tuple[int, int]]]:
    """(y, rng_state); `rng_state` = (seed, offset) reproduces the mask."""
    if p < 0.0 or p > 1.0:
        raise ValueError("dropout probability has to be between 0 and 1, but got {}".format(p))
    if not training or p == 0:
        return x, None
    if rng_state is None:
        rng_state = megalodon_ops.dropkey_philox_state(x.device, x.numel())
    return megalodon_ops.dropout(x, p, *rng_state), rng_state


def memory_efficient_dropout_bwd(y_grad: torch.Tensor, p: float, rng_state: Optional[Tuple[int, int]],
                                 noise: Optional[torch.Tensor] = None) -> torch.Tensor:
    if p == 0:
        assert rng_state is None
        return y_grad
    if noise is not None:
        return y_grad.mul(noise)
    return megalodon_ops.dropout(y_grad, p, *rng_state)
