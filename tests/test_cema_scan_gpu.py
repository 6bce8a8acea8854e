"""The chunked-recurrence CEMA kernels against the float64 oracle (closed-form
kernel + FFT convolution + carried-state bias + last state, and their autograd
gradients).  Bars: 2e-2 for bfloat16 / float16 tensors, 1e-4 for float32
tensors (the parameter gradients and the complex last state)."""
import math

import pytest
import torch

from conftest import rel_err
from megalodon_amd import extension as ops
from oracle import cema as ocema
from oracle import fftconv as offt

pytestmark = pytest.mark.gpu


def _params(D, N, seed):
    g = torch.Generator().manual_seed(seed)
    alpha = torch.sigmoid(torch.randn(D, N, 1, generator=g))
    delta = torch.sigmoid(torch.randn(D, N, 1, generator=g))
    theta = torch.rand(D, 1, 1, generator=g) * (2 * math.pi / N)
    q = torch.polar(1.0 - alpha * delta, theta * torch.arange(1, N + 1, dtype=torch.float32).view(1, N, 1))
    gam = torch.complex(torch.randn(D, N, generator=g), torch.randn(D, N, generator=g)) / math.sqrt(2 * N)
    omega = torch.randn(D, generator=g)
    return alpha, q, gam, omega


def _oracle_fwd(x, p, q, gam, omega, h0):
    L = x.shape[-1]
    lq = q.to(torch.complex128).log()
    k = ocema.ema_weight_fwd(p.double(), lq, gam.to(torch.complex128), L)
    want = offt.fftconv_fwd(x.double(), k) + x.double() * omega.double().view(1, -1, 1)
    if h0 is not None:
        want = want + ocema.ema_bias_fwd(lq, gam.to(torch.complex128), h0.to(torch.complex128), L)
    last = ocema.ema_hidden_fwd(x.double(), p.double(), lq, None if h0 is None else h0.to(torch.complex128))
    return want, last


SHAPES = [(1, 2, 16, 8), (2, 3, 16, 64), (1, 3, 16, 72), (2, 2, 5, 1000), (1, 4, 16, 4096), (2, 2, 16, 8200),
          (1, 3, 16, 16384), (1, 2, 16, 16392), (1, 5, 16, 32768), (1, 2, 16, 40000), (1, 2, 1, 2048),
          (1, 2, 16, 65536)]


@pytest.mark.parametrize("B,D,N,L", SHAPES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("state", [False, True])
def test_forward_matches_oracle(B, D, N, L, dtype, state):
    p, q, gam, omega = _params(D, N, 3 * L + D)
    g = torch.Generator().manual_seed(L)
    x = torch.randn(B, D, L, generator=g).to(dtype)
    h0 = torch.complex(torch.randn(B, D, N, generator=g), torch.randn(B, D, N, generator=g)) if state else None
    assert ops.cema_scan_supported(x.cuda(), N)
    y, last = ops.cema_scan_fwd(x.cuda(), p.cuda(), q.log().cuda(), gam.cuda(), omega.cuda(),
                                None if h0 is None else h0.cuda(), True)
    want, wlast = _oracle_fwd(x, p, q, gam, omega, h0)
    assert y.dtype == dtype and y.shape == x.shape
    assert rel_err(y, want) <= (1e-4 if dtype == torch.float32 else 2e-2)
    # the rounding of y aside, the values carry float32 accuracy: compare before rounding would need
    # a float32 output, so the last state (complex64, never rounded to 16 bits) stands for it
    assert last.shape == (B, D, N) and rel_err(last, wlast) <= 1e-4


def test_forward_without_skip_term_and_without_last_state():
    B, D, N, L = 2, 3, 16, 3000
    p, q, gam, omega = _params(D, N, 5)
    x = torch.randn(B, D, L, generator=torch.Generator().manual_seed(1)).bfloat16()
    y, last = ops.cema_scan_fwd(x.cuda(), p.cuda(), q.log().cuda(), gam.cuda(), None)
    want, _ = _oracle_fwd(x, p, q, gam, torch.zeros(D), None)
    assert last is None and rel_err(y, want) <= 2e-2


def test_unsupported_shapes_are_refused():
    x = torch.zeros(1, 2, 100, dtype=torch.bfloat16, device="cuda")   # L % 8 != 0
    assert not ops.cema_scan_supported(x, 16)
    assert ops.cema_scan_supported(torch.zeros(1, 2, 64, device="cuda"), 16)       # float32 rows
    assert ops.cema_scan_bwd_supported(torch.zeros(1, 2, 64, device="cuda"), 16)   # float32 rows: two bf16 pieces
    assert ops.cema_scan_bwd_supported(torch.zeros(1, 2, 64, dtype=torch.float16, device="cuda"), 16)
    assert ops.cema_scan_supported(torch.zeros(1, 2, 64, dtype=torch.bfloat16, device="cuda"), 17)   # two launches
    assert not ops.cema_scan_supported(torch.zeros(1, 2, 64, dtype=torch.bfloat16, device="cuda"), 33)
    p, q, gam, omega = _params(2, 16, 1)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        ops.cema_scan_fwd(x, p.cuda(), q.log().cuda(), gam.cuda(), omega.cuda())


BWD_SHAPES = [(1, 2, 16, 8), (2, 3, 16, 64), (1, 3, 16, 72), (2, 2, 5, 1000), (1, 4, 16, 4096), (3, 2, 16, 8200),
              (1, 3, 16, 16384), (1, 2, 16, 8264), (1, 3, 16, 32768), (1, 2, 16, 40000), (1, 2, 1, 2048)]


@pytest.mark.parametrize("B,D,N,L", BWD_SHAPES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_backward_matches_oracle(B, D, N, L, dtype):
    p, q, gam, omega = _params(D, N, 5 * L + D)
    g = torch.Generator().manual_seed(L + 1)
    x = torch.randn(B, D, L, generator=g).to(dtype)
    dy = torch.randn(B, D, L, generator=g).to(dtype)
    # bfloat16 rows in one launch, float16 / float32 rows in three launches on two bfloat16 pieces each
    assert ops.cema_scan_bwd_supported(x.cuda(), N)
    dx, dp, dq, dg, dw = ops.cema_scan_bwd(dy.cuda(), x.cuda(), p.cuda(), q.log().cuda(), gam.cuda(), omega.cuda())
    lq = q.to(torch.complex128).log()
    k = ocema.ema_weight_fwd(p.double(), lq, gam.to(torch.complex128), L)
    wdx, wdk = offt.fftconv_bwd(dy.double(), x.double(), k)
    wdp, wdq, wdg = ocema.ema_weight_bwd(wdk, p.double(), lq, gam.to(torch.complex128))
    assert dx.dtype == dtype
    assert rel_err(dx, wdx + dy.double() * omega.double().view(1, D, 1)) <= (1e-4 if dtype == torch.float32 else 2e-2)
    assert rel_err(dp, wdp.reshape(D, N)) <= 1e-4
    assert rel_err(dq, wdq.reshape(D, N)) <= 1e-4
    assert rel_err(dg, wdg.reshape(D, N)) <= 1e-4
    assert rel_err(dw, (dy.double() * x.double()).sum(dim=(0, 2))) <= 1e-4


@pytest.mark.parametrize("decay", ["slow", "fast", "mixed"])
def test_extreme_decay_rates(decay):
    """|q| within 1e-4 of 1 (states that sum ten thousand steps), |q| near 0 (powers that
    underflow inside a chunk) and both in one channel, forward with last state and backward."""
    B, D, N, L = 1, 3, 16, 16384
    g = torch.Generator().manual_seed(11)
    if decay == "slow":
        mag = 1.0 - 1e-4 * (1.0 + torch.rand(D, N, 1, generator=g))
    elif decay == "fast":
        mag = 1e-3 * (1.0 + torch.rand(D, N, 1, generator=g))
    else:
        mag = torch.where(torch.rand(D, N, 1, generator=g) < 0.5, torch.full((D, N, 1), 0.9999), torch.full((D, N, 1), 0.01))
    theta = torch.rand(D, 1, 1, generator=g) * (2 * math.pi / N)
    q = torch.polar(mag, theta * torch.arange(1, N + 1, dtype=torch.float32).view(1, N, 1))
    p = torch.rand(D, N, 1, generator=g)
    gam = torch.complex(torch.randn(D, N, generator=g), torch.randn(D, N, generator=g)) / math.sqrt(2 * N)
    omega = torch.randn(D, generator=g)
    x = torch.randn(B, D, L, generator=g).bfloat16()
    dy = torch.randn(B, D, L, generator=g).bfloat16()
    # The operators take log q, as the reference's do (fused_ops/ema_parameters.py:19 passes
    # q.log() in complex64).  Near |q| = 1 the float32 logarithm of the float32 q is itself
    # off by 6e-4 of the decay rate, so the oracle gets the same log q the kernel gets.
    lq32 = q.log()
    lq = lq32.to(torch.complex128)
    y, last = ops.cema_scan_fwd(x.cuda(), p.cuda(), lq32.cuda(), gam.cuda(), omega.cuda(), None, True)
    k = ocema.ema_weight_fwd(p.double(), lq, gam.to(torch.complex128), L)
    want = offt.fftconv_fwd(x.double(), k) + x.double() * omega.double().view(1, -1, 1)
    wlast = ocema.ema_hidden_fwd(x.double(), p.double(), lq, None)
    assert rel_err(y, want) <= 2e-2 and rel_err(last, wlast) <= 1e-4
    dx, dp, dq, dg, dw = ops.cema_scan_bwd(dy.cuda(), x.cuda(), p.cuda(), lq32.cuda(), gam.cuda(), omega.cuda())
    k = ocema.ema_weight_fwd(p.double(), lq, gam.to(torch.complex128), L)
    wdx, wdk = offt.fftconv_bwd(dy.double(), x.double(), k)
    wdp, wdq, wdg = ocema.ema_weight_bwd(wdk, p.double(), lq, gam.to(torch.complex128))
    assert rel_err(dx, wdx + dy.double() * omega.double().view(1, D, 1)) <= 2e-2
    assert rel_err(dp, wdp.reshape(D, N)) <= 1e-4
    assert rel_err(dq, wdq.reshape(D, N)) <= 1e-4
    assert rel_err(dg, wdg.reshape(D, N)) <= 1e-4


def _oracle_bwd(dy, x, p, q, gam, omega, h0):
    D, N = p.shape[0], p.shape[1]
    L = x.shape[-1]
    lq = q.to(torch.complex128).log()
    k = ocema.ema_weight_fwd(p.double(), lq, gam.to(torch.complex128), L)
    wdx, wdk = offt.fftconv_bwd(dy.double(), x.double(), k)
    wdp, wdq, wdg = ocema.ema_weight_bwd(wdk, p.double(), lq, gam.to(torch.complex128))
    wdx = wdx + dy.double() * omega.double().view(1, D, 1)
    wdq, wdg, wdh = wdq.reshape(D, N), wdg.reshape(D, N), None
    if h0 is not None:
        bq, bg, wdh = ocema.ema_bias_bwd(dy.double(), lq, gam.to(torch.complex128), h0.to(torch.complex128))
        wdq, wdg = wdq + bq.reshape(D, N), wdg + bg.reshape(D, N)
    return wdx, wdp.reshape(D, N), wdq, wdg, (dy.double() * x.double()).sum(dim=(0, 2)), wdh


@pytest.mark.parametrize("B,D,N,L", [(2, 3, 16, 64), (1, 2, 16, 8264), (3, 2, 7, 1000), (1, 3, 16, 32768)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_backward_with_carried_state(B, D, N, L, dtype):
    """The backward of a forward that had a carried state: the state's terms in dq and dgamma and
    its own gradient dh0 (ema_parameters.cc:100-117,158-188) from what the reverse scan carries to
    the start of the row."""
    p, q, gam, omega = _params(D, N, 7 * L + D)
    g = torch.Generator().manual_seed(L + 2)
    x = torch.randn(B, D, L, generator=g).to(dtype)
    dy = torch.randn(B, D, L, generator=g).to(dtype)
    h0 = torch.complex(torch.randn(B, D, N, generator=g), torch.randn(B, D, N, generator=g))
    dx, dp, dq, dg, dw, dh = ops.cema_scan_bwd(dy.cuda(), x.cuda(), p.cuda(), q.log().cuda(), gam.cuda(), omega.cuda(),
                                               h0.cuda())
    wdx, wdp, wdq, wdg, wdw, wdh = _oracle_bwd(dy, x, p, q, gam, omega, h0)
    assert dx.dtype == dtype and rel_err(dx, wdx) <= (1e-4 if dtype == torch.float32 else 2e-2)
    assert rel_err(dp, wdp) <= 1e-4 and rel_err(dq, wdq) <= 1e-4 and rel_err(dg, wdg) <= 1e-4
    assert rel_err(dw, wdw) <= 1e-4
    assert dh.shape == (B, D, N) and rel_err(dh, wdh) <= 1e-4


@pytest.mark.parametrize("N", [17, 24, 32])
def test_more_than_sixteen_modes(N):
    """The reference takes up to 32 modes (ema_parameters_kernel.cu:1026); the kernels hold 16, the
    modes are independent and their outputs add up: forward with state and last state, backward
    with the state's gradient."""
    B, D, L = 2, 3, 4096
    p, q, gam, omega = _params(D, N, 100 + N)
    g = torch.Generator().manual_seed(N)
    x = torch.randn(B, D, L, generator=g).bfloat16()
    dy = torch.randn(B, D, L, generator=g).bfloat16()
    h0 = torch.complex(torch.randn(B, D, N, generator=g), torch.randn(B, D, N, generator=g))
    assert ops.cema_scan_supported(x.cuda(), N) and ops.cema_scan_bwd_supported(x.cuda(), N)
    y, last = ops.cema_scan_fwd(x.cuda(), p.cuda(), q.log().cuda(), gam.cuda(), omega.cuda(), h0.cuda(), True)
    want, wlast = _oracle_fwd(x, p, q, gam, omega, h0)
    assert rel_err(y, want) <= 2e-2 and last.shape == (B, D, N) and rel_err(last, wlast) <= 1e-4
    dx, dp, dq, dg, dw, dh = ops.cema_scan_bwd(dy.cuda(), x.cuda(), p.cuda(), q.log().cuda(), gam.cuda(), omega.cuda(),
                                               h0.cuda())
    wdx, wdp, wdq, wdg, wdw, wdh = _oracle_bwd(dy, x, p, q, gam, omega, h0)
    assert rel_err(dx, wdx) <= 2e-2
    assert rel_err(dp, wdp) <= 1e-4 and rel_err(dq, wdq) <= 1e-4 and rel_err(dg, wdg) <= 1e-4
    assert rel_err(dw, wdw) <= 1e-4 and rel_err(dh, wdh) <= 1e-4


def test_layer_trains_through_a_carried_state():
    """MultiHeadComplexEMA with hx and compute_last_state under autograd on the recurrence kernels:
    gradients of x and hx from both outputs (the output's through the state terms of the backward,
    the last state's through ema_hidden's backward) against the oracle's operators."""
    from megalodon_amd.modules import MultiHeadComplexEMA
    B, D, N, L = 2, 8, 16, 2048
    torch.manual_seed(3)
    layer = MultiHeadComplexEMA(D, N).cuda().train()
    with torch.no_grad():
        layer.omega.normal_(0, 0.5)
    g = torch.Generator().manual_seed(9)
    x = torch.randn(B, D, L, generator=g).bfloat16()
    dy = torch.randn(B, D, L, generator=g).bfloat16()
    h0 = torch.complex(torch.randn(B, D, N, generator=g), torch.randn(B, D, N, generator=g))
    gh = torch.complex(torch.randn(B, D, N, generator=g), torch.randn(B, D, N, generator=g))
    xc, hc = x.cuda().requires_grad_(True), h0.cuda().requires_grad_(True)
    out, last = layer(xc, hc, True)
    assert out.dtype == torch.bfloat16 and last.shape == (B, D, N)
    torch.autograd.backward([out, last], [dy.cuda(), gh.cuda()])

    with torch.no_grad():
        p, q, gam = (t.cpu() for t in layer._calc_coeffs())
    p, q = p.reshape(D, N, 1), q.reshape(D, N, 1)
    omega = layer.omega.detach().cpu().reshape(D)
    want, wlast = _oracle_fwd(x, p, q, gam, omega, h0)
    assert rel_err(out, want) <= 2e-2 and rel_err(last, wlast) <= 1e-4
    wdx, _, _, _, _, wdh = _oracle_bwd(dy, x, p, q, gam, omega, h0)
    lq = q.to(torch.complex128).log()
    hdx, _, _, hdh = ocema.ema_hidden_bwd(gh, x.double(), p.double(), lq, h0)
    assert rel_err(xc.grad, wdx + hdx) <= 2e-2
    assert rel_err(hc.grad, wdh + hdh) <= 1e-4
    for prm in layer.parameters():
        assert prm.grad is not None and torch.isfinite(prm.grad).all()
