"""Parity of the HIP `ema_parameters` weight path against the float64 oracle.
Tolerance: rel err (max|a-b|/max|b|) <= 1e-4 in fp32, forward and gradients."""
import math

import pytest
import torch

from conftest import rel_err
from megalodon_amd import extension as ops
from megalodon_amd import synthetic
from megalodon_amd.fused_ops import ema_parameters
from oracle import cema

pytestmark = pytest.mark.gpu
TOL = 1e-4


def _case(D, N, seed):
    prm = synthetic.cema_params(D, N, seed)
    return prm["p"], prm["q"], prm["gamma"]


@pytest.mark.parametrize("D,N,L", [
    (1024, 16, 2048),    # config 0 (CEMA forward, fp32)
    (64, 16, 32768),     # config 1 length, fewer channels
    (7, 16, 1),
    (5, 16, 1000),       # ragged: not a multiple of the tile, unaligned rows
    (3, 16, 4099),
    (4, 1, 513),
    (4, 3, 2050),
    (2, 32, 3000),       # N > 16 path
    (2, 17, 70000),      # more than one slab of tiles
])
def test_weight_fwd_matches_oracle(D, N, L):
    p, q, gamma = _case(D, N, 100 + N + L % 97)
    lq = q.log()
    w, b, v = ops.ema_parameters_fwd(p.cuda(), lq.cuda(), gamma.cuda(), None, L)
    assert b is None and v is None
    assert w.shape == (D, L) and w.dtype == torch.float32
    want = cema.ema_weight_fwd(p, lq, gamma, L)
    assert rel_err(w, want) <= TOL


def test_weight_fwd_slow_decay_long_sequence_phase_accuracy():
    # |q| -> 1 with large angle: j*arg(q) reaches ~2e5 rad; direct fp32 phase would lose 1e-2
    D, N, L = 8, 16, 32768
    p = torch.full((D, N, 1), 0.5)
    rho = torch.full((D, N, 1), 0.99995)
    phi = torch.linspace(0.1, 6.2, D * N).view(D, N, 1)
    q = torch.polar(rho, phi)
    gamma = torch.complex(torch.ones(D, N), torch.ones(D, N)) * 0.25
    lq = q.log()
    w, _, _ = ops.ema_parameters_fwd(p.cuda(), lq.cuda(), gamma.cuda(), None, L)
    want = cema.ema_weight_fwd(p, lq, gamma, L)
    assert rel_err(w, want) <= TOL


@pytest.mark.parametrize("D,N,L", [
    (256, 16, 2048),
    (32, 16, 32768),
    (5, 16, 1000),
    (3, 16, 4099),
    (4, 3, 2051),
    (2, 32, 3000),
    (2, 16, 70001),
    (3, 16, 1),
])
def test_weight_bwd_matches_oracle(D, N, L):
    p, q, gamma = _case(D, N, 200 + N + L % 89)
    lq = q.log()
    g = torch.Generator().manual_seed(L)
    dw = torch.randn(D, L, generator=g)
    dp, dq, dg, dh = ops.ema_parameters_bwd(dw.cuda(), None, p.cuda(), lq.cuda(), gamma.cuda(), None, None)
    assert dh is None
    assert dp.shape == p.shape and dq.shape == lq.shape and dg.shape == gamma.shape
    wp, wq, wg = cema.ema_weight_bwd(dw, p, lq, gamma)
    assert rel_err(dp.reshape(D, N), wp) <= TOL
    assert rel_err(dq.reshape(D, N), wq) <= TOL
    assert rel_err(dg.reshape(D, N), wg) <= TOL


def test_autograd_function_grads_reach_p_q_gamma():
    D, N, L = 16, 16, 777
    p, q, gamma = _case(D, N, 9)
    pc = p.cuda().requires_grad_(True)
    qc = q.cuda().requires_grad_(True)
    gc = gamma.cuda().requires_grad_(True)
    w, b = ema_parameters(pc, qc, gc, None, L)
    assert b is None
    g = torch.Generator().manual_seed(1)
    dw = torch.randn(D, L, generator=g)
    w.backward(dw.cuda())
    wp, wq, wg = cema.ema_weight_bwd(dw, p, q.log(), gamma)
    assert rel_err(pc.grad.reshape(D, N), wp) <= TOL
    assert rel_err(qc.grad.reshape(D, N), wq) <= TOL
    assert rel_err(gc.grad.reshape(D, N), wg) <= TOL


def test_errors_are_loud():
    p, q, gamma = _case(2, 16, 1)
    with pytest.raises(RuntimeError):
        ops.ema_parameters_fwd(p, q.log(), gamma, None, 8)  # CPU tensors: no fallback
    with pytest.raises(RuntimeError):
        ops.ema_parameters_fwd(p.double().cuda(), q.log().cuda(), gamma.cuda(), None, 8)
    p40 = torch.rand(2, 40, 1).cuda()
    q40 = torch.polar(torch.rand(2, 40, 1) * 0.9, torch.rand(2, 40, 1)).cuda()
    g40 = torch.randn(2, 40, dtype=torch.complex64).cuda()
    with pytest.raises(RuntimeError, match="outside"):
        ops.ema_parameters_fwd(p40, q40.log(), g40, None, 8)


@pytest.mark.parametrize("D,N", [(5, 16), (64, 16), (7, 3), (33, 1), (4, 64)])
def test_fused_coefficients_match_oracle(D, N):
    """mega_cema_coeffs_fwd/bwd against the float64 restatement of
    _calc_coeffs and autograd over it (log q instead of q on the forward side,
    gradients w.r.t. q on the backward side, as the weight operator uses them)."""
    g = torch.Generator().manual_seed(D * 100 + N)
    alpha = torch.randn(D, N, 1, generator=g)
    delta = torch.randn(D, N, 1, generator=g)
    theta = torch.randn(D, 1, 1, generator=g)
    gamma = torch.randn(D, N, 2, generator=g)
    p, log_q, gh = ops.cema_coeffs_fwd(alpha.cuda(), delta.cuda(), theta.cuda(), gamma.cuda())
    a64, d64, t64, g64 = (t.double().requires_grad_(True) for t in (alpha, delta, theta, gamma))
    wp, wq, wg = cema.calc_coeffs(a64, d64, t64, g64, N)
    assert p.shape == (D, N, 1) and log_q.shape == (D, N, 1) and gh.shape == (D, N)
    assert rel_err(p, wp) <= 1e-6
    assert rel_err(torch.exp(log_q), wq) <= 1e-5
    assert rel_err(log_q.real, wq.abs().log()) <= 1e-5   # the phase is n theta_hat in (0, 2 pi), not the wrapped one
    assert float(log_q.imag.min()) > 0.0 and float(log_q.imag.max()) < 2 * math.pi
    assert rel_err(torch.view_as_real(gh), torch.view_as_real(wg)) <= 1e-6
    dp = torch.randn(D, N, 1, generator=g)
    dq = torch.view_as_complex(torch.randn(D, N, 1, 2, generator=g))
    dg = torch.view_as_complex(torch.randn(D, N, 2, generator=g))
    # PyTorch convention: backward with grad_output g gives dL/dRe + i dL/dIm for L = Re(sum conj(g) z)
    torch.autograd.backward([wp, wq, wg], [dp.double(), dq.to(torch.complex128), dg.to(torch.complex128)])
    got = ops.cema_coeffs_bwd(dp.cuda(), dq.cuda(), dg.cuda(), alpha.cuda(), delta.cuda(), theta.cuda())
    for name, a, b in zip(["dalpha", "ddelta", "dtheta", "dgamma"], got, (a64.grad, d64.grad, t64.grad, g64.grad)):
        assert a.shape == b.shape, name
        assert rel_err(a, b) <= 1e-5, name
