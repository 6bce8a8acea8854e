"""The chunked-recurrence form of the CEMA layer, checked on the CPU in float64.

The CEMA kernel is a sum of N damped complex exponentials, k[j] = Re sum_n c_n
q_n^j (csrc/ops/ema_parameters.cc:37-52), so `fftconv(x, k)` is a linear
recurrence with N complex states per channel
(complex_exponential_moving_average.py:127-147, ema_hidden.cc:31-61).  The HIP
kernels of csrc/cema_scan.hip evaluate it chunk by chunk as small matrix
products; this file states that algebra with plain tensor products, in the
same decomposition (chunks of T steps, local products, a scan over chunk
states), and checks it against the oracle built from the closed-form kernel
and the FFT convolution.  The GPU tests then compare the kernels with the same
oracle."""
import math

import pytest
import torch

from oracle import cema as ocema
from oracle import fftconv as offt

T = 64


def _params(D, N, seed):
    g = torch.Generator().manual_seed(seed)
    alpha = torch.sigmoid(torch.randn(D, N, generator=g, dtype=torch.float64))
    delta = torch.sigmoid(torch.randn(D, N, generator=g, dtype=torch.float64))
    theta = torch.rand(D, 1, generator=g, dtype=torch.float64) * (2 * math.pi / N)
    q = torch.polar(1.0 - alpha * delta, theta * torch.arange(1, N + 1, dtype=torch.float64))
    gam = torch.complex(torch.randn(D, N, generator=g, dtype=torch.float64),
                        torch.randn(D, N, generator=g, dtype=torch.float64)) / math.sqrt(2 * N)
    omega = torch.randn(D, generator=g, dtype=torch.float64)
    return alpha, q, gam, omega


def _chunks(row, T):
    """(..., L) -> (..., C, T), zero padded at the end."""
    L = row.shape[-1]
    C = -(-L // T)
    return torch.nn.functional.pad(row, (0, C * T - L)).reshape(*row.shape[:-1], C, T), C


def scan_forward(x, p, q, gam, omega, h0=None, T=T):
    """y (B, D, L) and the state after the last step (B, D, N), by chunks:
      S[c]   = p sum_j q^(T-1-j) x[c, j]                  local chunk state
      H[c]   = q^T H[c-1] + S[c],  H[-1] = h0             scan over chunks
      y[c,i] = sum_{j<=i} k[i-j] x[c,j] + Re sum_n gam_n q_n^(i+1) H_n[c-1] + omega x[c,i]"""
    B, D, L = x.shape
    N = q.shape[1]
    xc, C = _chunks(x, T)
    e = torch.arange(T + 1, dtype=torch.float64)
    qp = q.unsqueeze(-1) ** e                                   # (D, N, T+1): q^e
    cq = (p * gam).unsqueeze(-1) * qp[..., :T]                  # c q^l
    klocal = cq.real.sum(1)                                     # (D, T): k[0..T-1]
    idx = torch.arange(T)
    lag = idx.view(T, 1) - idx.view(1, T)                       # i - j
    Km = torch.where(lag >= 0, klocal[:, lag.clamp(min=0)], torch.zeros((), dtype=torch.float64))  # (D, T, T)
    Pm = p.unsqueeze(-1) * qp[..., :T].flip(-1)                 # (D, N, T): p q^(T-1-j)
    S = torch.einsum("bdcj,dnj->bdcn", xc.to(torch.complex128), Pm)
    H = torch.zeros(B, D, C + 1, N, dtype=torch.complex128)     # H[:, :, c+1] = state after chunk c
    if h0 is not None:
        H[:, :, 0] = h0
    qT = qp[..., T]
    for c in range(C):
        H[:, :, c + 1] = qT * H[:, :, c] + S[:, :, c]
    Qm = gam.unsqueeze(-1) * qp[..., 1:]                        # (D, N, T): gam q^(i+1)
    y = torch.einsum("dij,bdcj->bdci", Km, xc) + torch.einsum("dni,bdcn->bdci", Qm, H[:, :, :C]).real
    y = y.reshape(B, D, C * T)[..., :L] + omega.view(1, D, 1) * x
    # state at the true end of the row: the last chunk may be partial
    r = L - (C - 1) * T
    last = qp[..., r] * H[:, :, C - 1] + torch.einsum(
        "bdj,dnj->bdn", xc[:, :, C - 1, :r].to(torch.complex128), p.unsqueeze(-1) * qp[..., :r].flip(-1))
    return y, last


def scan_backward(dy, x, p, q, gam, omega, T=T):
    """dx and the per-channel sums the parameter gradients need, by chunks, in
    reverse time.  With c_n = p_n gam_n,
      A_n = sum_{t>=s} dy[t] x[s] q_n^(t-s),   B_n = dA_n / dq_n
    (S2 and S1 of ema_parameters.cc:80-98 with dk eliminated), and
      dp = Re(A gam), dq = conj(B p gam), dgam = conj(A p), domega = sum dy x.
    Chunk form (x is time-reversed inside a chunk so that one power matrix,
    q^i and i q^(i-1) for i < T, serves both streams; no division by q):
      G[c]  = sum_i dy[c,i] q^i,        G'[c] = sum_i dy[c,i] i q^(i-1)
      R[c]  = G[c] + q^T R[c+1]                            reverse-time state of dy at the chunk's start
      R'[c] = G'[c] + T q^(T-1) R[c+1] + q^T R'[c+1]
      X[c]  = sum_j' xrev[c,j'] q^j' (= sum_j x[c,j] q^(T-1-j)),   X'[c] = sum_j' xrev[c,j'] j' q^(j'-1)
      dx[c,j] = sum_{i>=j} k[i-j] dy[c,i] + Re sum_n c_n q_n^(T-j) R_n[c+1] + omega dy[c,j]
      A = sum_l q^l dkin[l] + q W,        W = sum_c X[c] R[c+1]
      B = sum_l l q^(l-1) dkin[l] + W + q sum_c (X'[c] R[c+1] + X[c] R'[c+1])
    with dkin[l] = sum_c sum_j x[c,j] dy[c,j+l] the within-chunk correlation:
    a pair (s in chunk c, t in a later chunk c') has
    q^(t-s) = q^(T-1-j) q q^((c'-c-1) T) q^i."""
    B_, D, L = x.shape
    xc, C = _chunks(x, T)
    dc, _ = _chunks(dy, T)
    e = torch.arange(T + 1, dtype=torch.float64)
    qp = q.unsqueeze(-1) ** e                                   # (D, N, T+1)
    P0 = qp[..., :T]                                            # q^i, i < T
    P0d = torch.cat([torch.zeros_like(P0[..., :1]), e[1:T] * qp[..., :T - 1]], dim=-1)   # i q^(i-1)
    G = torch.einsum("bdci,dni->bdcn", dc.to(torch.complex128), P0)
    Gd = torch.einsum("bdci,dni->bdcn", dc.to(torch.complex128), P0d)
    xrev = xc.flip(-1)
    X = torch.einsum("bdcj,dnj->bdcn", xrev.to(torch.complex128), P0)
    Xd = torch.einsum("bdcj,dnj->bdcn", xrev.to(torch.complex128), P0d)
    qT, qTd = qp[..., T], T * qp[..., T - 1]
    R = torch.zeros(B_, D, C + 1, q.shape[1], dtype=torch.complex128)    # R[C] = 0
    Rd = torch.zeros_like(R)
    for c in range(C - 1, -1, -1):
        R[:, :, c] = G[:, :, c] + qT * R[:, :, c + 1]
        Rd[:, :, c] = Gd[:, :, c] + qTd * R[:, :, c + 1] + qT * Rd[:, :, c + 1]
    cg = p * gam
    klocal = (cg.unsqueeze(-1) * qp[..., :T]).real.sum(1)       # (D, T)
    idx = torch.arange(T)
    lag = idx.view(1, T) - idx.view(T, 1)                       # i - j at [j, i]
    KmT = torch.where(lag >= 0, klocal[:, lag.clamp(min=0)], torch.zeros((), dtype=torch.float64))  # (D, j, i)
    Qd = cg.unsqueeze(-1) * qp[..., 1:].flip(-1)                # (D, N, T): c q^(T-j)
    dx = torch.einsum("dji,bdci->bdcj", KmT, dc) + torch.einsum("dnj,bdcn->bdcj", Qd, R[:, :, 1:]).real
    dx = dx.reshape(B_, D, C * T)[..., :L] + omega.view(1, D, 1) * dy
    # within-chunk correlation: the l-th diagonal of dy^T x summed over chunks and batch
    M = torch.einsum("bdci,bdcj->dij", dc, xc)                   # (D, i, j)
    dkin = torch.stack([torch.diagonal(M, offset=-l, dim1=1, dim2=2).sum(-1) for l in range(T)], dim=-1)  # (D, T)
    A_in = (dkin.unsqueeze(1) * P0).sum(-1)
    B_in = (dkin.unsqueeze(1) * P0d).sum(-1)
    W = (X * R[:, :, 1:]).sum(dim=(0, 2))
    Wd = (Xd * R[:, :, 1:] + X * Rd[:, :, 1:]).sum(dim=(0, 2))
    A = A_in + q * W
    Bq = B_in + W + q * Wd
    dp = (A * gam).real
    dq = (Bq * p * gam).conj()
    dgam = (A * p).conj()
    domega = dkin[:, 0]
    return dx, dp, dq, dgam, domega


@pytest.mark.parametrize("B,D,N,L", [(2, 3, 4, 200), (1, 2, 16, 64), (1, 2, 16, 1000), (2, 2, 3, 129), (1, 1, 16, 4096)])
def test_chunked_forward_equals_fft_convolution(B, D, N, L):
    p, q, gam, omega = _params(D, N, L)
    g = torch.Generator().manual_seed(L + 1)
    x = torch.randn(B, D, L, generator=g, dtype=torch.float64)
    k = ocema.ema_weight_fwd(p.unsqueeze(-1), q.log().unsqueeze(-1), gam, L)
    want = offt.fftconv_fwd(x, k) + x * omega.view(1, D, 1)
    got, last = scan_forward(x, p, q, gam, omega)
    assert torch.allclose(got, want, atol=1e-10, rtol=1e-10)
    assert torch.allclose(last, ocema.ema_hidden_fwd(x, p.unsqueeze(-1), q.log().unsqueeze(-1), None), atol=1e-10)


@pytest.mark.parametrize("L", [64, 100, 515])
def test_chunked_forward_with_initial_state(L):
    B, D, N = 2, 3, 8
    p, q, gam, omega = _params(D, N, 7)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(B, D, L, generator=g, dtype=torch.float64)
    h0 = torch.complex(torch.randn(B, D, N, generator=g, dtype=torch.float64),
                       torch.randn(B, D, N, generator=g, dtype=torch.float64))
    lq = q.log().unsqueeze(-1)
    k = ocema.ema_weight_fwd(p.unsqueeze(-1), lq, gam, L)
    want = offt.fftconv_fwd(x, k) + x * omega.view(1, D, 1) + ocema.ema_bias_fwd(lq, gam, h0, L)
    got, last = scan_forward(x, p, q, gam, omega, h0)
    assert torch.allclose(got, want, atol=1e-10, rtol=1e-10)
    assert torch.allclose(last, ocema.ema_hidden_fwd(x, p.unsqueeze(-1), lq, h0), atol=1e-10)


@pytest.mark.parametrize("B,D,N,L", [(2, 3, 4, 200), (1, 2, 16, 64), (1, 2, 16, 1000), (3, 2, 5, 129)])
def test_chunked_backward_equals_oracle_gradients(B, D, N, L):
    p, q, gam, omega = _params(D, N, 11 * L)
    g = torch.Generator().manual_seed(L + 5)
    x = torch.randn(B, D, L, generator=g, dtype=torch.float64)
    dy = torch.randn(B, D, L, generator=g, dtype=torch.float64)
    lq = q.log().unsqueeze(-1)
    k = ocema.ema_weight_fwd(p.unsqueeze(-1), lq, gam, L)
    wdx, wdk = offt.fftconv_bwd(dy, x, k)
    wdp, wdq, wdg = ocema.ema_weight_bwd(wdk, p.unsqueeze(-1), lq, gam)
    dx, dp, dq, dgam, dom = scan_backward(dy, x, p, q, gam, omega)
    assert torch.allclose(dx, wdx + dy * omega.view(1, D, 1), atol=1e-10, rtol=1e-10)
    assert torch.allclose(dp, wdp.reshape(D, N), atol=1e-9, rtol=1e-9)
    assert torch.allclose(dq, wdq.reshape(D, N), atol=1e-8, rtol=1e-9)
    assert torch.allclose(dgam, wdg.reshape(D, N), atol=1e-9, rtol=1e-9)
    assert torch.allclose(dom, (dy * x).sum(dim=(0, 2)), atol=1e-10)
