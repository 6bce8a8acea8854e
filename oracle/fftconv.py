"""Oracle for the causal FFT convolution (float64).

Follows megalodon/modules/fused_ops/fftconv.py:30-75 (`_fftconv_fwd`,
`_fftconv_bwd`): zero-pad to 2N with N = next power of two >= L, rfft, multiply,
irfft, crop to L; backward through flipped sequences.
"""
from __future__ import annotations

import numpy as np
import torch


def _pow2(L: int) -> int:
    return L if (L & (L - 1)) == 0 else (1 << L.bit_length())


def fftconv_fwd(x, k):
    """y = irfft(rfft(x, 2N) * rfft(k, 2N))[..., :L]   (fftconv.py:30-50).
    x: (B, D, L), k: (D, L).  Returns float64."""
    L = x.shape[-1]
    N = _pow2(L)
    x = x.double()
    k = k.double()
    x_f = torch.fft.rfft(x, n=2 * N)
    k_f = torch.fft.rfft(k, n=2 * N, norm="forward")
    return torch.fft.irfft(x_f * k_f, n=2 * N, norm="forward")[..., :L]


def fftconv_bwd(dy, x, k):
    """(dx, dk) restating fftconv.py:53-75 (x_f, k_f recomputed from x, k)."""
    L = dy.shape[-1]
    N = _pow2(L)
    dy = dy.double()
    x_f = torch.fft.rfft(x.double(), n=2 * N)
    k_f = torch.fft.rfft(k.double(), n=2 * N, norm="forward")
    dy_f = torch.fft.rfft(dy.flip(dims=(-1,)), n=2 * N)
    dx = torch.fft.irfft(dy_f * k_f, n=2 * N, norm="forward")[..., :L].flip(dims=(-1,))
    dk = torch.fft.irfft((dy_f * x_f).sum(dim=0), n=2 * N)[..., :L].flip(dims=(-1,))
    return dx, dk


def causal_conv_bruteforce(x, k):
    """y[b,d,t] = sum_{s<=t} k[d,t-s] x[b,d,s] by explicit loops (tiny sizes)."""
    x = np.asarray(x, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    B, D, L = x.shape
    y = np.zeros_like(x)
    for b in range(B):
        for d in range(D):
            for t in range(L):
                s = 0.0
                for u in range(t + 1):
                    s += k[d, t - u] * x[b, d, u]
                y[b, d, t] = s
    return y
