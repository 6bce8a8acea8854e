"""`MultiHeadComplexEMA` with the reference's constructor, parameters and forward
(megalodon/modules/complex_exponential_moving_average.py:42-150), minus the
`megalodon.distributed` look-ups: model-parallel world size is 1, so
``dim_per_partition == embed_dim`` and the theta permutation is drawn locally
instead of being broadcast (:21-26).  On the GPU the layer runs as a chunked
recurrence (fused_ops/cema_scan.py) wherever its kernels take the case --
rows of a length that is a multiple of 8, at most 32 modes, with or without
gradients, carried state and last state; MEGA_CEMA_FFT=1 in the environment
keeps everything on the kernel-row + FFT-convolution operators that the
remaining cases (other lengths) use."""
from typing import Optional, Tuple
import math
import os

import torch
from torch import nn

from .. import extension as megalodon_ops
from ..fused_ops import (cema_kernel, cema_scan, cema_scan_applicable, cema_scan_state, ema_hidden, ema_parameters,
                         fftconv_residual)


@torch.no_grad()
def _reset_parameters(alpha, delta, theta, gamma, omega, embed_dim):
    """Initial values as in the reference (:64-98): narrow normal logits for the
    decay pair; base frequencies sigmoid(theta) = D^(-i/D), i = 1..D in random
    order (log-spaced between 1/D and 1); real N(0, 1) mixing weights; a
    truncated normal skip weight."""
    alpha.normal_(0.0, 0.2)
    delta.normal_(0.0, 0.2)
    order = (torch.randperm(embed_dim) + 1).to(torch.float32)
    base = torch.exp(-order * (math.log(embed_dim) / embed_dim))
    theta.copy_(torch.logit(base).view(embed_dim, 1, 1))
    gamma[..., 0].normal_(0.0, 1.0)
    gamma[..., 1].zero_()
    nn.init.trunc_normal_(omega, mean=0.0, std=0.25, a=-1.0, b=1.0)


class MultiHeadComplexEMA(nn.Module):
    """Complex Exponential Moving Average layer."""

    def __init__(self, embed_dim, ndim=16):
        super().__init__()
        self.embed_dim = embed_dim
        self.ndim = ndim
        self.scale = math.sqrt(1.0 / self.ndim)
        self.dim_per_partition = embed_dim

        self.alpha = nn.Parameter(torch.Tensor(self.dim_per_partition, ndim, 1))
        self.delta = nn.Parameter(torch.Tensor(self.dim_per_partition, ndim, 1))
        self.theta = nn.Parameter(torch.Tensor(self.dim_per_partition, 1, 1))
        self.gamma = nn.Parameter(torch.Tensor(self.dim_per_partition, ndim, 2))
        self.omega = nn.Parameter(torch.Tensor(self.dim_per_partition, 1))
        self._coeffs = None
        self._init_parameters()

    def _init_parameters(self):
        _reset_parameters(self.alpha, self.delta, self.theta, self.gamma, self.omega, self.embed_dim)

    def _calc_coeffs(self):
        """(p, q, gamma_hat) in float32: p = sigmoid(alpha) (D, N, 1);
        q = (1 - p sigmoid(delta)) exp(i n base), n = 1..N, with base =
        sigmoid(theta) 2 pi / N (D, N, 1) complex; gamma_hat = gamma / sqrt(N)
        (D, N) complex (:100-117)."""
        self._coeffs = None
        self._coeffs_kernel = None
        n_modes = self.ndim
        p = torch.sigmoid(self.alpha.float())
        base = torch.sigmoid(self.theta.float()) * (2 * math.pi / n_modes)
        harmonics = torch.arange(1, n_modes + 1, dtype=base.dtype, device=base.device).view(1, n_modes, 1)
        q = torch.polar(1.0 - p * torch.sigmoid(self.delta.float()), base * harmonics)
        return p, q, torch.view_as_complex(self.gamma.float()) * self.scale

    def coeffs(self):
        if self.training:
            return self._calc_coeffs()
        if self._coeffs is None:
            self._coeffs = self._calc_coeffs()
        return self._coeffs

    @torch.no_grad()
    def _kernel_coeffs(self):
        """(p, log q, gamma_hat) from the coefficient kernel, for the branches that need no gradient;
        cached in evaluation mode beside (and dropped with) the coefficients of `coeffs()`."""
        make = lambda: megalodon_ops.cema_coeffs_fwd(self.alpha.float(), self.delta.float(), self.theta.float(),
                                                     self.gamma.float())
        if self.training:
            return make()
        self.coeffs()
        if getattr(self, "_coeffs_kernel", None) is None:
            self._coeffs_kernel = make()
        return self._coeffs_kernel

    def forward(
        self,
        x: torch.Tensor,
        hx: Optional[torch.Tensor] = None,
        compute_last_state: bool = False,
    ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        # B x D x L
        bsz, _, seq_len = x.size()
        if self.training:
            # the reference's training forward goes through _calc_coeffs(), which drops the
            # coefficients cached for evaluation (:100-101,119-125); every branch below does the same
            self._coeffs = None
            self._coeffs_kernel = None
        stateless = hx is None and not compute_last_state
        needs_grad = torch.is_grad_enabled() and (x.requires_grad or any(t.requires_grad for t in self.parameters())
                                                  or (hx is not None and hx.requires_grad))
        if self.alpha.is_cuda and os.environ.get("MEGA_CEMA_FFT") is None:
            # the layer as a chunked recurrence on the matrix cores (no kernel row, no
            # transform, any length in one launch): bfloat16 / float16 rows with or without
            # gradients, float32 rows and carried states where no gradient is wanted
            if stateless and cema_scan_applicable(x, self.ndim, needs_grad):
                out = cema_scan(x, self.alpha.float(), self.delta.float(), self.theta.float(), self.gamma.float(),
                                self.omega)
                return out, None
            if not stateless and needs_grad and cema_scan_applicable(x, self.ndim, True):
                # carried state in, last state out, all differentiable (dh0 included)
                return cema_scan_state(x, self.alpha.float(), self.delta.float(), self.theta.float(),
                                       self.gamma.float(), self.omega, hx, compute_last_state)
            if not stateless and not needs_grad and cema_scan_applicable(x, self.ndim, False):
                # log q from the coefficient kernel, the one the stateless branch uses: a prefill
                # and its carried continuation see the same decay rates
                p, log_q, gamma = self._kernel_coeffs()
                return megalodon_ops.cema_scan_fwd(x, p, log_q, gamma, self.omega, hx, compute_last_state)
        if stateless and self.alpha.is_cuda:
            # no carried state: coefficients and kernel as one autograd node
            # (two launches per direction instead of the coefficient graph)
            k, b = cema_kernel(self.alpha.float(), self.delta.float(), self.theta.float(), self.gamma.float(),
                               seq_len), None
            p = q = None
        else:
            p, q, gamma = self.coeffs()
            k, b = ema_parameters(p, q, gamma, hx, seq_len)
        # fftconv(x, k) + x * omega, the skip term folded into the convolution's
        # output pass (the reference adds `residual = x * self.omega` afterwards)
        output = fftconv_residual(x, k, self.omega)
        if b is not None:
            output = output + b.to(output)
        # compute the last hidden state
        h = ema_hidden(x, p, q, hx) if compute_last_state else None
        return output, h

    def extra_repr(self) -> str:
        return 'edim={} ({}), ndim={}'.format(self.embed_dim, self.dim_per_partition, self.ndim)
