"""`fftconv` autograd op (mirror of megalodon/modules/fused_ops/fftconv.py:9-27).

The reference saves the spectra ``(x_f, k_f)`` for backward; `fftconv` saves
``(x, k)`` and the backward kernel recomputes the transforms on chip, while
`fftconv_residual` (the op the CEMA layer uses) keeps the two spectra whenever
the shape runs on the matrix-core path."""
from typing import Tuple

import torch
from torch.autograd.function import FunctionCtx

from ..extension import (fftconv_bwd, fftconv_fwd, fftconv_residual_bwd, fftconv_residual_bwd_saved,
                         fftconv_residual_fwd, fftconv_residual_fwd_saving, fftconv_spectrum_bytes)


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


def fused_fftconv_fwd(x: torch.Tensor, k: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(y, x_saved, k_saved) with the call pattern of the reference's
    ``fused_fftconv_fwd(x, k) -> (y, x_f, k_f)`` (fused_ops/fftconv.py:79-93).
    The two saved tensors are what ``fused_fftconv_bwd`` takes back; here they
    are x and k themselves (the backward kernel recomputes the transforms on
    chip), not complex spectra."""
    return fftconv_fwd(x, k), x, k


def fused_fftconv_bwd(y_grad: torch.Tensor, x_saved: torch.Tensor, k_saved: torch.Tensor,
                      k_dtype: torch.dtype) -> Tuple[torch.Tensor, torch.Tensor]:
    """(dx, dk) from the pair ``fused_fftconv_fwd`` returned
    (fused_ops/fftconv.py:96-106); dk has dtype ``k_dtype``."""
    return fftconv_bwd(y_grad, x_saved, k_saved, k_dtype)


class FFTConvResidualFunc(torch.autograd.Function):
    """``fftconv(x, k) + x * omega`` as one op: the two lines around the
    convolution in MultiHeadComplexEMA.forward
    (megalodon/modules/complex_exponential_moving_average.py:136-146) without the
    two extra passes over the activations.  The result has the dtype of x."""

    @staticmethod
    def forward(ctx: FunctionCtx, x: torch.Tensor, k: torch.Tensor, omega: torch.Tensor) -> torch.Tensor:
        # 16-bit rows on the matrix-core path keep the spectra of x and k for
        # the backward pass, as the reference keeps x_f and k_f
        # (fused_ops/fftconv.py:21-28); other shapes keep x and k themselves
        ctx.k_dtype = k.dtype
        x = x.contiguous()  # the CEMA layer hands in a transposed view
        ctx.spectra = (x.is_cuda and x.dim() == 3 and fftconv_spectrum_bytes(x.dtype, *x.shape) > 0
                       and x.data_ptr() % 16 == 0)
        if ctx.spectra:
            y, spec_x, spec_k = fftconv_residual_fwd_saving(x, k, omega)
            ctx.save_for_backward(spec_x, spec_k, omega)
        else:
            y = fftconv_residual_fwd(x, k, omega)
            ctx.save_for_backward(x, k, omega)
        return y

    @staticmethod
    def backward(ctx: FunctionCtx, y_grad: torch.Tensor):
        if ctx.spectra:
            spec_x, spec_k, omega = ctx.saved_tensors
            dx, dk, dw = fftconv_residual_bwd_saved(y_grad, spec_x, spec_k, omega)
        else:
            x, k, omega = ctx.saved_tensors
            dx, dk, dw = fftconv_residual_bwd(y_grad, x, k, omega)
        return dx, dk.to(ctx.k_dtype), dw.to(omega.dtype).view_as(omega)


fftconv_residual = FFTConvResidualFunc.apply
