"""Pins the carried-state parts of the CEMA oracle (oracle/cema.py: ema_bias_*,
ema_hidden_*): the EMA recurrence they must reproduce, autograd through the
closed forms, and the reference's own CPU operators (oracle/_ref)."""
import math

import pytest
import torch

from oracle import cema, native


def _case(B, D, N, L, seed, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    p = torch.sigmoid(torch.randn(D, N, generator=g, dtype=torch.float64))
    rho = 1.0 - p * torch.sigmoid(torch.randn(D, N, generator=g, dtype=torch.float64))
    q = torch.polar(rho, torch.rand(D, N, generator=g, dtype=torch.float64) * 2 * math.pi)
    gamma = torch.complex(torch.randn(D, N, generator=g, dtype=torch.float64),
                          torch.randn(D, N, generator=g, dtype=torch.float64))
    h = torch.complex(torch.randn(B, D, N, generator=g, dtype=torch.float64),
                      torch.randn(B, D, N, generator=g, dtype=torch.float64))
    x = torch.randn(B, D, L, generator=g, dtype=torch.float64)
    return p, q, gamma, h, x


def test_recurrence_reproduced_by_weight_bias_and_hidden():
    """h_t = q h_(t-1) + p x_t, y_t = Re(gamma . h_t) from a carried h_0: the
    outputs are conv(x, w) + b and the final state is ema_hidden."""
    B, D, N, L = 2, 3, 4, 41
    p, q, gamma, h0, x = _case(B, D, N, L, 0)
    hh, ys = h0.clone(), []
    for t in range(L):
        hh = q * hh + p * x[:, :, t].unsqueeze(-1)
        ys.append((gamma * hh).real.sum(-1))
    ys = torch.stack(ys, -1)
    w = cema.ema_weight_fwd(p, q.log(), gamma, L)
    conv = torch.zeros(B, D, L, dtype=torch.float64)
    for t in range(L):
        for s in range(t + 1):
            conv[:, :, t] += w[:, t - s] * x[:, :, s]
    b = cema.ema_bias_fwd(q.log(), gamma, h0, L)
    assert (conv + b - ys).abs().max() < 1e-12
    assert (cema.ema_hidden_fwd(x, p, q.log(), h0) - hh).abs().max() < 1e-12
    # without a carried state the recurrence starts from zero
    hz = torch.zeros_like(h0)
    for t in range(L):
        hz = q * hz + p * x[:, :, t].unsqueeze(-1)
    assert (cema.ema_hidden_fwd(x, p, q.log(), None) - hz).abs().max() < 1e-12


def test_splitting_a_sequence_with_carried_state():
    """Two halves with the state handed over equal the whole sequence."""
    B, D, N, L = 2, 2, 3, 30
    p, q, gamma, _, x = _case(B, D, N, L, 1)
    lq = q.log()
    w = cema.ema_weight_fwd(p, lq, gamma, L)
    full = torch.zeros(B, D, L, dtype=torch.float64)
    for t in range(L):
        for s in range(t + 1):
            full[:, :, t] += w[:, t - s] * x[:, :, s]
    L1 = 13
    h1 = cema.ema_hidden_fwd(x[:, :, :L1], p, lq, None)
    x2 = x[:, :, L1:]
    L2 = L - L1
    second = torch.zeros(B, D, L2, dtype=torch.float64)
    for t in range(L2):
        for s in range(t + 1):
            second[:, :, t] += w[:, t - s] * x2[:, :, s]
    second = second + cema.ema_bias_fwd(lq, gamma, h1, L2)
    assert (second - full[:, :, L1:]).abs().max() < 1e-12
    h2 = cema.ema_hidden_fwd(x2, p, lq, h1)
    assert (h2 - cema.ema_hidden_fwd(x, p, lq, None)).abs().max() < 1e-12


def test_backward_formulas_match_autograd():
    B, D, N, L = 2, 3, 4, 29
    p, q, gamma, h, x = _case(B, D, N, L, 2)
    xr, pr, qr, hr = (t.clone().requires_grad_() for t in (x, p, q, h))
    y = cema.ema_hidden_fwd(xr, pr, qr.log(), hr)
    dy = torch.complex(torch.randn(B, D, N, dtype=torch.float64), torch.randn(B, D, N, dtype=torch.float64))
    y.backward(dy)
    dx, dp, dq, dh = cema.ema_hidden_bwd(dy, x, p, q.log(), h)
    for got, want in ((dx, xr.grad), (dp, pr.grad), (dq, qr.grad), (dh, hr.grad)):
        assert (got - want).abs().max() <= 1e-10 * want.abs().max()
    dx2, dp2, dq2, dh2 = cema.ema_hidden_bwd(dy, x, p, q.log(), None)
    assert dh2 is None and (dx2 - dx).abs().max() == 0 and (dp2 - dp).abs().max() == 0
    qr, gr, hr = (t.clone().requires_grad_() for t in (q, gamma, h))
    b = cema.ema_bias_fwd(qr.log(), gr, hr, L)
    db = torch.randn(B, D, L, dtype=torch.float64)
    b.backward(db)
    dq, dg, dh = cema.ema_bias_bwd(db, q.log(), gamma, h)
    for got, want in ((dq, qr.grad), (dg, gr.grad), (dh, hr.grad)):
        assert (got - want).abs().max() <= 1e-10 * want.abs().max()


@pytest.mark.skipif(native.ref() is None, reason="oracle/_ref not built (needs /root/reference)")
def test_reference_cpp_cpu_operators_match_oracle():
    """EMAParametersCPUFwd/Bwd with a carried state and EMAHiddenCPUFwd/Bwd, compiled
    from the reference's sources, against the float64 restatement (float32 tolerance)."""
    lib = native.ref()

    def close(a, b, tol=2e-4):
        return (a.to(torch.complex128) - b.to(torch.complex128)).abs().max() <= tol * b.abs().max()

    for B, D, N, L, seed in [(2, 4, 16, 130, 5), (1, 3, 4, 33, 6), (3, 2, 1, 17, 7)]:
        p, q, gamma, h, x = _case(B, D, N, L, seed)
        p, q, gamma, h, x = p.float(), q.to(torch.complex64), gamma.to(torch.complex64), h.to(torch.complex64), x.float()
        lq = q.log()
        assert close(native.ema_bias_fwd(lib, p, lq, gamma, h, L), cema.ema_bias_fwd(lq, gamma, h, L))
        db = torch.randn(B, D, L, generator=torch.Generator().manual_seed(seed))
        for got, want in zip(native.ema_bias_bwd(lib, db, p, lq, gamma, h), cema.ema_bias_bwd(db, lq, gamma, h)):
            assert close(got, want)
        for hh in (h, None):
            assert close(native.ema_hidden_fwd(lib, x, p, lq, hh), cema.ema_hidden_fwd(x, p, lq, hh))
            dy = torch.randn(B, D, N, dtype=torch.complex64, generator=torch.Generator().manual_seed(seed + 1))
            got = native.ema_hidden_bwd(lib, dy, x, p, lq, hh)
            want = cema.ema_hidden_bwd(dy, x, p, lq, hh)
            for gt, wt in zip(got, want):
                assert (gt is None) == (wt is None)
                if gt is not None:
                    assert close(gt, wt)
