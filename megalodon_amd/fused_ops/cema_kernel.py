"""Convolution kernel of the CEMA layer straight from its raw parameters:
``k = ema_parameters(*_calc_coeffs(), None, L)[0]`` of
megalodon/modules/complex_exponential_moving_average.py:100-117,134 as one
autograd node with two launches per direction (coefficients, weight) instead
of the ~30 elementwise kernels of the coefficient graph."""
from typing import Tuple

import torch
from torch.autograd.function import FunctionCtx

from .. import extension as megalodon_ops


class CEMAKernelFunc(torch.autograd.Function):

    @staticmethod
    def forward(ctx: FunctionCtx, alpha: torch.Tensor, delta: torch.Tensor, theta: torch.Tensor,
                gamma: torch.Tensor, length: int) -> torch.Tensor:
        p, log_q, gamma_hat = megalodon_ops.cema_coeffs_fwd(alpha, delta, theta, gamma)
        weight, _, _ = megalodon_ops.ema_parameters_fwd(p, log_q, gamma_hat, None, length)
        ctx.save_for_backward(alpha, delta, theta, p, log_q, gamma_hat)
        return weight

    @staticmethod
    def backward(ctx: FunctionCtx, weight_grad: torch.Tensor) -> Tuple[torch.Tensor, ...]:
        alpha, delta, theta, p, log_q, gamma_hat = ctx.saved_tensors
        dp, dq, dg, _ = megalodon_ops.ema_parameters_bwd(weight_grad, None, p, log_q, gamma_hat, None, None)
        dalpha, ddelta, dtheta, dgamma = megalodon_ops.cema_coeffs_bwd(dp, dq, dg, alpha, delta, theta)
        return dalpha, ddelta, dtheta, dgamma, None


cema_kernel = CEMAKernelFunc.apply
