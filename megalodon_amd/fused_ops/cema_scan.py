"""The CEMA layer without a carried state as one autograd node over its raw
parameters: the lines
    p, q, gamma = self.coeffs()
    k, b = ema_parameters(p, q, gamma, None, L)
    out = fftconv(x, k) + x * self.omega
of megalodon/modules/complex_exponential_moving_average.py:127-147, evaluated
as a chunked recurrence (csrc/cema_scan.hip): two launches forward
(coefficients, recurrence), two backward; neither the kernel row k nor dk nor
any spectrum exists."""
from typing import Tuple

import torch
from torch.autograd.function import FunctionCtx

from .. import extension as megalodon_ops


class CEMAScanFunc(torch.autograd.Function):

    @staticmethod
    def forward(ctx: FunctionCtx, x: torch.Tensor, alpha: torch.Tensor, delta: torch.Tensor, theta: torch.Tensor,
                gamma: torch.Tensor, omega: torch.Tensor) -> torch.Tensor:
        p, log_q, gamma_hat = megalodon_ops.cema_coeffs_fwd(alpha, delta, theta, gamma)
        y, _ = megalodon_ops.cema_scan_fwd(x, p, log_q, gamma_hat, omega)
        ctx.save_for_backward(x, alpha, delta, theta, p, log_q, gamma_hat, omega)
        return y

    @staticmethod
    def backward(ctx: FunctionCtx, y_grad: torch.Tensor) -> Tuple[torch.Tensor, ...]:
        x, alpha, delta, theta, p, log_q, gamma_hat, omega = ctx.saved_tensors
        dx, dp, dq, dg, dw = megalodon_ops.cema_scan_bwd(y_grad, x, p, log_q, gamma_hat, omega)
        dalpha, ddelta, dtheta, dgamma = megalodon_ops.cema_coeffs_bwd(dp, dq, dg, alpha, delta, theta)
        return dx, dalpha, ddelta, dtheta, dgamma, dw.to(omega.dtype).view_as(omega)


cema_scan = CEMAScanFunc.apply


class CEMAScanStateFunc(torch.autograd.Function):
    """The same layer with a carried state and / or the last state wanted:
        k, b = ema_parameters(p, q, gamma, hx, L);  out = fftconv(x, k) + x * omega + b
        h = ema_hidden(x, p, q, hx)
    (complex_exponential_moving_average.py:131-147) as one node returning (out, h).  The backward of
    `out` is the recurrence's backward with the state's terms (ema_parameters.cc:158-188); a gradient
    that arrives at `h` goes through ema_hidden's backward (ema_hidden.cc:63-159)."""

    @staticmethod
    def forward(ctx: FunctionCtx, x, alpha, delta, theta, gamma, omega, hx, compute_last_state: bool):
        p, log_q, gamma_hat = megalodon_ops.cema_coeffs_fwd(alpha, delta, theta, gamma)
        y, h = megalodon_ops.cema_scan_fwd(x, p, log_q, gamma_hat, omega, hx, compute_last_state)
        ctx.save_for_backward(x, alpha, delta, theta, p, log_q, gamma_hat, omega, hx)
        return y, h

    @staticmethod
    def backward(ctx: FunctionCtx, y_grad, h_grad):
        x, alpha, delta, theta, p, log_q, gamma_hat, omega, hx = ctx.saved_tensors
        if y_grad is None:
            y_grad = torch.zeros_like(x)
        res = megalodon_ops.cema_scan_bwd(y_grad.contiguous(), x, p, log_q, gamma_hat, omega, hx)
        dx, dp, dq, dg, dw = res[:5]
        dh = res[5] if hx is not None else None
        if h_grad is not None:
            _, moments = megalodon_ops.ema_hidden_fwd(x, p, log_q, hx)
            dx2, dp2, dq2, dh2 = megalodon_ops.ema_hidden_bwd(h_grad, x, p, log_q, hx, moments)
            dx = (dx.float() + dx2.float()).to(dx.dtype)
            dp = dp + dp2.reshape(dp.shape)
            dq = dq + dq2.reshape(dq.shape)
            if dh is not None:
                dh = dh + dh2.reshape(dh.shape)
        dalpha, ddelta, dtheta, dgamma = megalodon_ops.cema_coeffs_bwd(dp, dq, dg, alpha, delta, theta)
        if dh is not None:
            dh = dh.reshape(hx.shape).to(hx.dtype)
        return dx, dalpha, ddelta, dtheta, dgamma, dw.to(omega.dtype).view_as(omega), dh, None


cema_scan_state = CEMAScanStateFunc.apply


def cema_scan_applicable(x: torch.Tensor, ndim: int, needs_grad: bool) -> bool:
    """The recurrence kernels take bfloat16 / float16 / float32 rows of a length that
    is a multiple of 8 with at most 32 modes (16 per launch), forward and backward;
    the backward runs float16 and float32 rows through their bfloat16 pieces."""
    if needs_grad:
        return megalodon_ops.cema_scan_bwd_supported(x, ndim)
    return megalodon_ops.cema_scan_supported(x, ndim)
