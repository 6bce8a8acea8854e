"""Pins the FFT-convolution oracle (oracle/fftconv.py): brute force, numpy
convolution, the EMA recurrence (no FFT involved) and autograd."""
import numpy as np
import pytest
import torch

from conftest import rel_err
from oracle import cema, fftconv


@pytest.mark.parametrize("B,D,L", [(2, 3, 1), (1, 2, 7), (2, 2, 32), (1, 3, 50), (1, 1, 129)])
def test_fwd_matches_bruteforce_and_numpy(B, D, L):
    g = torch.Generator().manual_seed(L)
    x = torch.randn(B, D, L, generator=g, dtype=torch.float64)
    k = torch.randn(D, L, generator=g, dtype=torch.float64)
    y = fftconv.fftconv_fwd(x, k).numpy()
    bf = fftconv.causal_conv_bruteforce(x.numpy(), k.numpy())
    assert np.allclose(y, bf, atol=1e-11)
    for b in range(B):
        for d in range(D):
            assert np.allclose(y[b, d], np.convolve(x[b, d].numpy(), k[d].numpy())[:L], atol=1e-11)


def test_fwd_equals_ema_recurrence():
    """conv with k = Re sum p*gamma*q^j equals h_t = q h_{t-1} + p x_t, y = Re(gamma . h)."""
    g = torch.Generator().manual_seed(3)
    B, D, N, L = 2, 3, 4, 50
    p = torch.rand(D, N, generator=g, dtype=torch.float64)
    q = torch.polar(torch.rand(D, N, generator=g, dtype=torch.float64) * 0.95,
                    torch.rand(D, N, generator=g, dtype=torch.float64) * 6.28)
    gamma = torch.complex(torch.randn(D, N, generator=g, dtype=torch.float64),
                          torch.randn(D, N, generator=g, dtype=torch.float64))
    omega = torch.randn(D, 1, generator=g, dtype=torch.float64)
    x = torch.randn(B, D, L, generator=g, dtype=torch.float64)
    k = cema.ema_weight_fwd(p, q.log(), gamma, L)
    out = fftconv.fftconv_fwd(x, k) + x * omega
    rec = cema.cema_forward(x, p, q, gamma, omega)
    assert torch.allclose(out, rec, atol=1e-11)


@pytest.mark.parametrize("B,D,L", [(2, 3, 9), (3, 2, 50), (1, 1, 64)])
def test_bwd_matches_autograd_over_bruteforce_sum(B, D, L):
    g = torch.Generator().manual_seed(L + 1)
    x = torch.randn(B, D, L, generator=g, dtype=torch.float64, requires_grad=True)
    k = torch.randn(D, L, generator=g, dtype=torch.float64, requires_grad=True)
    dy = torch.randn(B, D, L, generator=g, dtype=torch.float64)
    # explicit Toeplitz formulation: y[t] = sum_s K[t, s] x[s], K[t, s] = k[t-s] (t >= s)
    idx = torch.arange(L).view(L, 1) - torch.arange(L).view(1, L)
    K = torch.where(idx >= 0, k[:, idx.clamp(min=0)], torch.zeros((), dtype=torch.float64))
    y = torch.einsum("dts,bds->bdt", K, x)
    y.backward(dy)
    dx, dk = fftconv.fftconv_bwd(dy, x.detach(), k.detach())
    assert torch.allclose(dx, x.grad, atol=1e-10)
    assert torch.allclose(dk, k.grad, atol=1e-10)
    # correlation identities: dx[t] = sum_{s>=t} dy[s] k[s-t]; dk[j] = sum_b sum_{t>=j} dy[t] x[t-j]
    dxb = np.zeros((B, D, L))
    dkb = np.zeros((D, L))
    xn, kn, dyn = x.detach().numpy(), k.detach().numpy(), dy.numpy()
    for t in range(L):
        for s in range(t, L):
            dxb[:, :, t] += dyn[:, :, s] * kn[None, :, s - t]
    for j in range(L):
        for t in range(j, L):
            dkb[:, j] += (dyn[:, :, t] * xn[:, :, t - j]).sum(0)
    assert np.allclose(dx.numpy(), dxb, atol=1e-10)
    assert np.allclose(dk.numpy(), dkb, atol=1e-10)


@pytest.mark.parametrize("L,nb,S", [(100, 2, 56), (37, 3, 16), (64, 4, 16), (50, 2, 32)])
def test_long_row_block_decomposition_with_the_oracle_as_one_launch(L, nb, S):
    """The host-side cutting of rows longer than one launch (heads and tails of
    block pairs, tails as heads of reversed blocks), with the oracle standing in
    for the launch: equal to the oracle on the whole row, forward and backward."""
    from megalodon_amd import extension as ops
    g = torch.Generator().manual_seed(L)
    x = torch.randn(2, 3, L, generator=g, dtype=torch.float64)
    k = torch.randn(3, L, generator=g, dtype=torch.float64)
    dy = torch.randn(2, 3, L, generator=g, dtype=torch.float64)
    y = ops._fftconv_long_fwd(x, k, blocks=(nb, S), head=fftconv.fftconv_fwd)
    assert rel_err(y, fftconv.fftconv_fwd(x, k)) < 1e-6   # the sums over terms are float32
    dx, dk = ops._fftconv_long_bwd(dy, x, k, blocks=(nb, S), head_bwd=fftconv.fftconv_bwd)
    wdx, wdk = fftconv.fftconv_bwd(dy, x, k)
    assert rel_err(dx, wdx) < 1e-6 and rel_err(dk, wdk) < 1e-6


def test_long_row_block_sizes_fit_one_launch():
    from megalodon_amd import extension as ops
    top = ops.fftconv_max_length()
    for L in (top + 1, top + 7, 40000, 2 * top, 2 * top + 1, 100003, 8 * top, 8 * top + 5):
        nb, S = ops._long_blocks(L)
        assert nb >= 2 and S % 8 == 0 and S <= top and nb * S >= L > (nb - 1) * S
