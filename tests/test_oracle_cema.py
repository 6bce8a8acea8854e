"""Pins the CEMA oracle (oracle/cema.py) without the reference: closed forms,
invariants, autograd and finite differences.  The reference ships no vectors
for this path."""
import math

import numpy as np
import pytest
import torch

from oracle import cema


def _params(D, N, seed):
    g = torch.Generator().manual_seed(seed)
    p = torch.sigmoid(torch.randn(D, N, generator=g, dtype=torch.float64))
    rho = 1.0 - p * torch.sigmoid(torch.randn(D, N, generator=g, dtype=torch.float64))
    phi = torch.rand(D, N, generator=g, dtype=torch.float64) * 2 * math.pi
    q = torch.polar(rho, phi)
    gamma = torch.complex(torch.randn(D, N, generator=g, dtype=torch.float64),
                          torch.randn(D, N, generator=g, dtype=torch.float64))
    return p, q, gamma


def test_coeffs_direct_formulas():
    g = torch.Generator().manual_seed(0)
    D, N = 5, 4
    alpha = torch.randn(D, N, 1, generator=g)
    delta = torch.randn(D, N, 1, generator=g)
    theta = torch.randn(D, 1, 1, generator=g)
    gamma = torch.randn(D, N, 2, generator=g)
    p, q, gh = cema.calc_coeffs(alpha, delta, theta, gamma, N)
    for d in range(D):
        for n in range(N):
            a = 1 / (1 + math.exp(-alpha[d, n, 0].item()))
            de = 1 / (1 + math.exp(-delta[d, n, 0].item()))
            th = 1 / (1 + math.exp(-theta[d, 0, 0].item())) * 2 * math.pi / N * (n + 1)
            assert abs(p[d, n, 0].item() - a) < 1e-12
            qq = (1 - a * de) * complex(math.cos(th), math.sin(th))
            assert abs(complex(q[d, n, 0]) - qq) < 1e-12
            gg = complex(gamma[d, n, 0].item(), gamma[d, n, 1].item()) / math.sqrt(N)
            assert abs(complex(gh[d, n]) - gg) < 1e-7


def test_weight_geometric_special_case():
    # N=1, theta=0: k[j] = p*gamma_re*rho^j (real geometric sequence)
    p = torch.tensor([[0.3]], dtype=torch.float64)
    rho = 0.9
    q = torch.tensor([[complex(rho, 0.0)]], dtype=torch.complex128)
    gamma = torch.tensor([[complex(1.7, -0.4)]], dtype=torch.complex128)
    w = cema.ema_weight_fwd(p, q.log(), gamma, 50)
    want = 0.3 * 1.7 * rho ** np.arange(50)
    assert np.allclose(w[0].numpy(), want, rtol=1e-13, atol=0)


def test_weight_first_tap_and_phase_invariance_and_loops():
    p, q, gamma = _params(3, 4, 1)
    lq = q.log()
    w = cema.ema_weight_fwd(p, lq, gamma, 33)
    assert torch.allclose(w[:, 0], (p * gamma).real.sum(-1), atol=1e-13)
    w2 = cema.ema_weight_fwd(p, lq + 2j * math.pi, gamma, 33)
    assert torch.allclose(w, w2, atol=1e-10)
    wl = cema.ema_weight_fwd_loops(p.numpy(), lq.numpy(), gamma.numpy(), 33)
    assert np.allclose(w.numpy(), wl, atol=1e-13)
    # direct powers: sum_n Re(c q^j)
    j = np.arange(33)
    direct = ((p * gamma).numpy()[..., None] * q.numpy()[..., None] ** j).real.sum(1)
    assert np.allclose(w.numpy(), direct, atol=1e-12)


def test_weight_bwd_matches_autograd_wrt_q():
    """dq/dgamma follow PyTorch's conjugate convention, dq is w.r.t. q."""
    p, q, gamma = _params(4, 5, 2)
    L = 40
    g = torch.Generator().manual_seed(5)
    dw = torch.randn(4, L, generator=g, dtype=torch.float64)
    p_ = p.clone().requires_grad_(True)
    q_ = q.clone().requires_grad_(True)
    g_ = gamma.clone().requires_grad_(True)
    j = torch.arange(L, dtype=torch.float64)
    w = ((p_ * g_).unsqueeze(-1) * q_.unsqueeze(-1) ** j).real.sum(1)
    w.backward(dw)
    dp, dq, dg = cema.ema_weight_bwd(dw, p, q.log(), gamma)
    assert torch.allclose(dp, p_.grad, atol=1e-11)
    assert torch.allclose(dq, q_.grad, atol=1e-10)
    assert torch.allclose(dg, g_.grad, atol=1e-11)


def test_weight_bwd_finite_differences():
    p, q, gamma = _params(2, 3, 3)
    L = 17
    g = torch.Generator().manual_seed(6)
    dw = torch.randn(2, L, generator=g, dtype=torch.float64)
    dp, dq, dg = cema.ema_weight_bwd(dw, p, q.log(), gamma)

    def loss(p_, q_, g_):
        return (cema.ema_weight_fwd(p_, q_.log(), g_, L) * dw).sum().item()

    eps = 1e-6
    for d in range(2):
        for n in range(3):
            e = torch.zeros_like(p)
            e[d, n] = eps
            fd = (loss(p + e, q, gamma) - loss(p - e, q, gamma)) / (2 * eps)
            assert abs(fd - dp[d, n].item()) < 1e-6
            ec = torch.zeros_like(q)
            ec[d, n] = eps
            fr = (loss(p, q + ec, gamma) - loss(p, q - ec, gamma)) / (2 * eps)
            fi = (loss(p, q + 1j * ec, gamma) - loss(p, q - 1j * ec, gamma)) / (2 * eps)
            assert abs(complex(fr, fi) - complex(dq[d, n])) < 1e-5
            fr = (loss(p, q, gamma + ec) - loss(p, q, gamma - ec)) / (2 * eps)
            fi = (loss(p, q, gamma + 1j * ec) - loss(p, q, gamma - 1j * ec)) / (2 * eps)
            assert abs(complex(fr, fi) - complex(dg[d, n])) < 1e-6


# ---- compiled checkers: the C restatement and the reference's own C++ CPU path ----
from oracle import native


def _f32_case(D, N, seed):
    p, q, gamma = _params(D, N, seed)
    return p.float(), q.to(torch.complex64).log(), gamma.to(torch.complex64)


def test_c_port_matches_float64_oracle():
    lib = native.port()
    p, lq, gamma = _f32_case(6, 16, 11)
    L = 300
    w = native.ema_weight_fwd(lib, "oracle_", p, lq, gamma, L)
    want = cema.ema_weight_fwd(p, lq, gamma, L)
    assert (w.double() - want).abs().max() / want.abs().max() < 2e-5
    g = torch.Generator().manual_seed(3)
    dw = torch.randn(6, L, generator=g)
    dp, dq, dg = native.ema_weight_bwd(lib, "oracle_", dw, p, lq, gamma)
    wp, wq, wg = cema.ema_weight_bwd(dw, p, lq, gamma)
    assert (dp.double() - wp).abs().max() / wp.abs().max() < 1e-4
    assert (dq.to(torch.complex128) - wq).abs().max() / wq.abs().max() < 1e-4
    assert (dg.to(torch.complex128) - wg).abs().max() / wg.abs().max() < 1e-4


@pytest.mark.skipif(native.ref() is None, reason="oracle/_ref not built (needs /root/reference)")
def test_reference_cpp_cpu_path_matches_oracle():
    """The reference's EMAParametersCPUFwd/Bwd (compiled from its own sources)
    against the float64 restatement, float32 tolerance."""
    lib = native.ref()
    for D, N, L, seed in [(5, 16, 257, 1), (3, 4, 64, 2), (2, 1, 33, 3)]:
        p, lq, gamma = _f32_case(D, N, seed)
        w = native.ema_weight_fwd(lib, "ref_", p, lq, gamma, L)
        want = cema.ema_weight_fwd(p, lq, gamma, L)
        assert (w.double() - want).abs().max() / want.abs().max() < 2e-5
        g = torch.Generator().manual_seed(seed)
        dw = torch.randn(D, L, generator=g)
        dp, dq, dg = native.ema_weight_bwd(lib, "ref_", dw, p, lq, gamma)
        wp, wq, wg = cema.ema_weight_bwd(dw, p, lq, gamma)
        assert (dp.double() - wp).abs().max() / wp.abs().max() < 1e-4
        assert (dq.to(torch.complex128) - wq).abs().max() / wq.abs().max() < 1e-4
        assert (dg.to(torch.complex128) - wg).abs().max() / wg.abs().max() < 1e-4
