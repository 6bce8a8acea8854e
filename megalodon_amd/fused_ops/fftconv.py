"""`fftconv` autograd op (mirror of megalodon/modules/fused_ops/fftconv.py:9-27).

The reference saves the spectra ``(x_f, k_f)`` for backward; this op saves
``(x, k)`` and the backward kernel recomputes the transforms on chip."""
from typing import Tuple

import torch
from torch.autograd.function import FunctionCtx

from ..extension import fftconv_bwd, fftconv_fwd


class FFTConvFunc(torch.autograd.Function):

    @staticmethod
    def forward(ctx: FunctionCtx, x: torch.Tensor, k: torch.Tensor) -> torch.Tensor:
        y = fftconv_fwd(x, k)
        ctx.save_for_backward(x, k)
        ctx.k_dtype = k.dtype  # k_dtype is not a torch.Tensor
        return y

    @staticmethod
    def backward(ctx: FunctionCtx, y_grad: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        x, k = ctx.saved_tensors
        return fftconv_bwd(y_grad, x, k, ctx.k_dtype)


fftconv = FFTConvFunc.apply
