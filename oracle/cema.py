"""Oracle for the CEMA coefficient and convolution-kernel path (float64).

Follows
  megalodon/modules/complex_exponential_moving_average.py:100-117 (coefficients)
  megalodon/csrc/ops/ema_parameters.cc:17-52   (weight forward)
  megalodon/csrc/ops/ema_parameters.cc:80-98   (weight backward)
  megalodon/modules/fused_ops/ema_parameters.py:19 (log_q = q.log())
"""
from __future__ import annotations

import math

import numpy as np
import torch


def calc_coeffs(alpha, delta, theta, gamma, ndim):
    """(p, q, gamma_hat) from raw parameters.

    alpha, delta: (D, N, 1); theta: (D, 1, 1); gamma: (D, N, 2).
    complex_exponential_moving_average.py:100-117:
      theta_hat = sigmoid(theta) * 2*pi/N * [1..N];  p = sigmoid(alpha)
      q = polar(1 - sigmoid(alpha) sigmoid(delta), theta_hat)
      gamma_hat = view_as_complex(gamma) * sqrt(1/N)
    """
    alpha = alpha.double()
    delta = delta.double()
    theta = theta.double()
    gamma = gamma.double()
    th = torch.sigmoid(theta) * (2.0 * math.pi / ndim)
    wavelets = torch.arange(1, ndim + 1, dtype=torch.float64).view(1, ndim)
    th = wavelets.unsqueeze(2) * th
    a = torch.sigmoid(alpha)
    d = torch.sigmoid(delta)
    p = a
    q = torch.polar(1.0 - a * d, th)
    g = torch.view_as_complex(gamma.contiguous()) * math.sqrt(1.0 / ndim)
    return p, q, g


def ema_weight_fwd(p, log_q, gamma, L):
    """w[d, j] = sum_n Re(p*gamma * exp(log_q * j)) (ema_parameters.cc:37-52).

    p: (D, N) or (D, N, 1) real; log_q, gamma: complex, same leading shape.
    Returns float64 (D, L).  Works on torch tensors (autograd flows).
    """
    D = p.shape[0]
    p = p.reshape(D, -1).to(torch.float64)
    log_q = log_q.reshape(D, -1).to(torch.complex128)
    gamma = gamma.reshape(D, -1).to(torch.complex128)
    j = torch.arange(L, dtype=torch.float64)
    c = p * gamma  # (D, N)
    qw = torch.exp(log_q.unsqueeze(-1) * j)  # (D, N, L)
    return (c.unsqueeze(-1) * qw).real.sum(dim=1)


def ema_weight_fwd_loops(p, log_q, gamma, L):
    """Scalar-loop restatement of ema_parameters.cc:37-52 for tiny cases."""
    p = np.asarray(p, dtype=np.float64)
    log_q = np.asarray(log_q, dtype=np.complex128)
    gamma = np.asarray(gamma, dtype=np.complex128)
    D, N = p.shape
    w = np.zeros((D, L))
    for d in range(D):
        for j in range(L):
            s = 0.0
            for n in range(N):
                qw = np.exp(log_q[d, n] * j)
                s += (p[d, n] * gamma[d, n] * qw).real
            w[d, j] = s
    return w


def ema_weight_bwd(dw, p, log_q, gamma):
    """(dp, dq, dgamma) from dw, restating ema_parameters.cc:80-98.

      sum1 = sum_i dw[i] * i * q^(i-1)   (i = 0 term is 0)
      sum2 = sum_i dw[i] * q^i
      dp = Re(sum2*gamma); dq = conj(sum1*p*gamma); dgamma = conj(sum2*p)
    """
    D = p.shape[0]
    p = p.reshape(D, -1).to(torch.float64)
    log_q = log_q.reshape(D, -1).to(torch.complex128)
    gamma = gamma.reshape(D, -1).to(torch.complex128)
    dw = dw.to(torch.float64)
    L = dw.shape[-1]
    i = torch.arange(L, dtype=torch.float64)
    q = torch.exp(log_q)
    qw1 = torch.exp(log_q.unsqueeze(-1) * (i - 1.0))  # q^(i-1)
    qw1[..., 0] = 0.0
    qw2 = qw1 * q.unsqueeze(-1)
    qw2[..., 0] = 1.0
    dwc = dw.unsqueeze(1).to(torch.complex128)
    sum1 = (dwc * qw1 * i).sum(-1)
    sum2 = (dwc * qw2).sum(-1)
    dp = (sum2 * gamma).real
    dq = torch.conj(sum1 * p * gamma)
    dgamma = torch.conj(sum2 * p)
    return dp, dq, dgamma


def cema_forward(x, p, q, gamma, omega):
    """out = causal_conv(x, k) + x*omega with k from (p, q, gamma)
    (complex_exponential_moving_average.py:127-147, hx=None branch).
    x: (B, D, L) ; omega: (D, 1).  Direct O(L^2)-free evaluation through the
    EMA recurrence h_t = q h_{t-1} + p x_t, y_t = Re(gamma . h_t)."""
    B, D, L = x.shape
    x = x.double()
    p = p.reshape(D, -1).double()
    q = q.reshape(D, -1).to(torch.complex128)
    gamma = gamma.reshape(D, -1).to(torch.complex128)
    h = torch.zeros(B, D, p.shape[1], dtype=torch.complex128)
    ys = []
    for t in range(L):
        h = q * h + p * x[:, :, t].unsqueeze(-1)
        ys.append((gamma * h).real.sum(-1))
    y = torch.stack(ys, dim=-1)
    return y + x * omega.double().reshape(1, D, 1)


# ---- carried state: bias of ema_parameters and the last hidden state ---------------
def _c128(t, *shape):
    return t.reshape(*shape).to(torch.complex128)


def ema_bias_fwd(log_q, gamma, h, L):
    """b[b, d, j] = sum_n Re(exp(log_q (j + 1)) gamma h[b, d, n]) (ema_parameters.cc:56-77).
    h: (B, D, N) complex.  Returns float64 (B, D, L)."""
    B, D, N = h.shape
    lq, g, hh = _c128(log_q, D, N), _c128(gamma, D, N), h.to(torch.complex128)
    j = torch.arange(1, L + 1, dtype=torch.float64)
    qw = torch.exp(lq.unsqueeze(-1) * j)  # (D, N, L): q^(j+1)
    return ((g.unsqueeze(-1) * qw).unsqueeze(0) * hh.unsqueeze(-1)).real.sum(dim=2)


def ema_bias_bwd(db, log_q, gamma, h):
    """(dq, dgamma, dh) contributions of the bias, restating RowwiseEMABiasCPUBwd
    and its caller (ema_parameters.cc:100-117, 158-188):
      sum1 = sum_i db[i] (i + 1) q^i,  sum2 = sum_i db[i] q^(i + 1)
      dq += conj(sum1 gamma h), dgamma += conj(sum2 h) (summed over the batch), dh = conj(sum2 gamma)."""
    B, D, N = h.shape
    L = db.shape[-1]
    lq, g, hh = _c128(log_q, D, N), _c128(gamma, D, N), h.to(torch.complex128)
    i = torch.arange(L, dtype=torch.float64)
    qw1 = torch.exp(lq.unsqueeze(-1) * i)          # q^i
    qw2 = qw1 * torch.exp(lq).unsqueeze(-1)        # q^(i+1)
    dbc = db.to(torch.float64).to(torch.complex128).unsqueeze(2)  # (B, D, 1, L)
    sum1 = (dbc * qw1 * (i + 1.0)).sum(-1)         # (B, D, N)
    sum2 = (dbc * qw2).sum(-1)
    return torch.conj(sum1 * g * hh).sum(0), torch.conj(sum2 * hh).sum(0), torch.conj(sum2 * g)


def ema_hidden_fwd(x, p, log_q, h):
    """y[b, d, n] = p sum_j exp(log_q (L - 1 - j)) x[b, d, j] (+ exp(log_q L) h)
    (ema_hidden.cc:16-62).  Returns complex128 (B, D, N)."""
    B, D, L = x.shape
    pp = p.reshape(D, -1).to(torch.float64)
    N = pp.shape[1]
    lq = _c128(log_q, D, N)
    e = torch.arange(L - 1, -1, -1, dtype=torch.float64)       # L - 1 - j
    qw = torch.exp(lq.unsqueeze(-1) * e)                       # (D, N, L)
    y = (qw.unsqueeze(0) * x.to(torch.float64).unsqueeze(2)).sum(-1) * pp
    if h is not None:
        y = y + torch.exp(lq * float(L)) * h.to(torch.complex128)
    return y


def ema_hidden_bwd(dy, x, p, log_q, h):
    """(dx, dp, dq, dh) restating ema_hidden.cc:64-159 (PyTorch conjugate convention)."""
    B, D, L = x.shape
    pp = p.reshape(D, -1).to(torch.float64)
    N = pp.shape[1]
    lq = _c128(log_q, D, N)
    q = torch.exp(lq)
    dyc = torch.conj(dy.to(torch.complex128))                   # (B, D, N)
    xx = x.to(torch.float64)
    e = torch.arange(L - 1, -1, -1, dtype=torch.float64)       # L - 1 - j
    qw2 = torch.exp(lq.unsqueeze(-1) * e)                      # q^(L-1-j)
    qw1 = torch.exp(lq.unsqueeze(-1) * (e - 1.0))              # q^(L-j-2), unused at j = L-1
    qw1[..., L - 1] = 0.0
    dx = ((dyc * pp).unsqueeze(-1) * qw2.unsqueeze(0)).real.sum(dim=2)
    xq2 = (qw2.unsqueeze(0) * xx.unsqueeze(2)).sum(-1)         # sum_j x q^(L-1-j)
    xq1 = (qw1.unsqueeze(0) * (xx * e).unsqueeze(2)).sum(-1)   # sum_j x (L-1-j) q^(L-j-2)
    dp = (dyc * xq2).real.sum(0)
    sum2 = (dyc * pp * xq1).sum(0)
    dh = None
    if h is not None:
        hh = h.to(torch.complex128)
        qw = torch.exp(lq * float(L - 1))
        sum2 = sum2 + (dyc * hh).sum(0) * qw * float(L)
        dh = torch.conj(dyc * qw * q)
    return dx, dp, torch.conj(sum2), dh
