"""The double-precision flavours of the CEMA operators against the float64 oracle.

The reference instantiates `ema_parameters`, `ema_hidden` and `fftconv` for
float64 / complex128 too (ema_parameters_kernel.cu:1227, fftconv_kernel.cu:468-476).
Here those dtypes run the defining sums in double on the GPU.  Tolerance: rel err
(max|a-b|/max|b|) <= 1e-10 -- both sides are float64; what differs is the order of
the sums and, for the convolution, the oracle's FFT against the direct sum."""
import math

import pytest
import torch

from conftest import rel_err
from megalodon_amd import extension as ops
from oracle import cema
from oracle import fftconv as offt

pytestmark = pytest.mark.gpu
TOL = 1e-10


def _params(B, D, N, L, seed):
    g = torch.Generator().manual_seed(seed)
    p = torch.sigmoid(torch.randn(D, N, 1, generator=g, dtype=torch.float64))
    rho = 1.0 - p * torch.sigmoid(torch.randn(D, N, 1, generator=g, dtype=torch.float64))
    q = torch.polar(rho, torch.rand(D, N, 1, generator=g, dtype=torch.float64) * 2 * math.pi)
    gamma = torch.randn(D, N, dtype=torch.complex128, generator=g)
    h = torch.randn(B, D, N, dtype=torch.complex128, generator=g)
    x = torch.randn(B, D, L, generator=g, dtype=torch.float64)
    return p, q, gamma, h, x


@pytest.mark.parametrize("B,D,N,L", [(2, 5, 16, 300), (1, 3, 4, 1), (2, 2, 16, 4099), (1, 2, 32, 700)])
def test_ema_parameters_with_bias(B, D, N, L):
    p, q, gamma, h, _ = _params(B, D, N, L, 3 * L + B)
    lq = q.log()
    w, b, v = ops.ema_parameters_fwd(p.cuda(), lq.cuda(), gamma.cuda(), h.cuda(), L)
    assert w.dtype == torch.float64 and w.shape == (D, L) and b.dtype == torch.float64 and v is None
    assert rel_err(w, cema.ema_weight_fwd(p, lq, gamma, L)) <= TOL
    assert rel_err(b, cema.ema_bias_fwd(lq, gamma, h, L)) <= TOL
    g = torch.Generator().manual_seed(L)
    dw = torch.randn(D, L, generator=g, dtype=torch.float64)
    db = torch.randn(B, D, L, generator=g, dtype=torch.float64)
    dp, dq, dg, dh = ops.ema_parameters_bwd(dw.cuda(), db.cuda(), p.cuda(), lq.cuda(), gamma.cuda(), h.cuda(), None)
    assert dp.dtype == torch.float64 and dq.dtype == torch.complex128 and dg.dtype == torch.complex128
    wp, wq, wg = cema.ema_weight_bwd(dw, p, lq, gamma)
    bq, bg, bh = cema.ema_bias_bwd(db, lq, gamma, h)
    assert rel_err(dp.reshape(D, N), wp) <= TOL
    assert rel_err(dq.reshape(D, N), wq + bq) <= TOL
    assert rel_err(dg.reshape(D, N), wg + bg) <= TOL
    assert rel_err(dh, bh) <= TOL
    # without a state: the weight path alone
    dp2, dq2, dg2, dh2 = ops.ema_parameters_bwd(dw.cuda(), None, p.cuda(), lq.cuda(), gamma.cuda(), None, None)
    assert dh2 is None and rel_err(dq2.reshape(D, N), wq) <= TOL and rel_err(dg2.reshape(D, N), wg) <= TOL


def test_precisions_must_agree():
    p, q, gamma, _, _ = _params(1, 2, 4, 8, 1)
    with pytest.raises(RuntimeError, match="complex128"):
        ops.ema_parameters_fwd(p.cuda(), q.log().to(torch.complex64).cuda(), gamma.cuda(), None, 8)
    with pytest.raises(RuntimeError, match="complex64"):
        ops.ema_parameters_fwd(p.float().cuda(), q.log().cuda(), gamma.cuda(), None, 8)


@pytest.mark.parametrize("B,D,N,L", [(2, 5, 16, 300), (1, 3, 4, 1), (2, 2, 16, 4099)])
@pytest.mark.parametrize("with_h", [True, False])
def test_ema_hidden(B, D, N, L, with_h):
    p, q, gamma, h, x = _params(B, D, N, L, 5 * L + B)
    lq = q.log()
    hh = h if with_h else None
    y, v = ops.ema_hidden_fwd(x.cuda(), p.cuda(), lq.cuda(), None if hh is None else hh.cuda())
    assert y.shape == (B, D, N) and y.dtype == torch.complex128
    assert rel_err(y, cema.ema_hidden_fwd(x, p, lq, hh)) <= TOL
    dy = torch.randn(B, D, N, dtype=torch.complex128, generator=torch.Generator().manual_seed(L))
    dx, dp, dq, dh = ops.ema_hidden_bwd(dy.cuda(), x.cuda(), p.cuda(), lq.cuda(),
                                        None if hh is None else hh.cuda(), v)
    wx, wp, wq, wh = cema.ema_hidden_bwd(dy, x, p, lq, hh)
    assert dx.dtype == torch.float64
    assert rel_err(dx, wx) <= TOL and rel_err(dp.reshape(D, N), wp) <= TOL and rel_err(dq.reshape(D, N), wq) <= TOL
    assert (dh is None) == (wh is None)
    if dh is not None:
        assert rel_err(dh, wh) <= TOL


@pytest.mark.parametrize("B,D,L", [(2, 3, 50), (1, 4, 256), (2, 3, 257), (1, 2, 4097), (3, 2, 1000)])
def test_convolution_and_residual_variant(B, D, L):
    g = torch.Generator().manual_seed(L + B)
    x = torch.randn(B, D, L, generator=g, dtype=torch.float64)
    k = torch.randn(D, L, generator=g, dtype=torch.float64) / math.sqrt(L)
    dy = torch.randn(B, D, L, generator=g, dtype=torch.float64)
    omega = torch.randn(D, 1, generator=g, dtype=torch.float64)
    y = ops.fftconv_fwd(x.cuda(), k.cuda())
    assert y.dtype == torch.float64 and y.shape == x.shape
    want = offt.fftconv_fwd(x, k)
    assert rel_err(y, want) <= TOL
    # causality to the last bit: the direct sum never touches later samples
    x2 = x.clone()
    x2[..., L // 2:] += 1.0
    assert torch.equal(ops.fftconv_fwd(x2.cuda(), k.cuda())[..., :L // 2], y[..., :L // 2])
    dx, dk = ops.fftconv_bwd(dy.cuda(), x.cuda(), k.cuda(), torch.float64)
    wdx, wdk = offt.fftconv_bwd(dy, x, k)
    assert dk.dtype == torch.float64 and rel_err(dx, wdx) <= TOL and rel_err(dk, wdk) <= TOL
    yr = ops.fftconv_residual_fwd(x.cuda(), k.cuda(), omega.cuda())
    assert rel_err(yr, want + omega.view(1, D, 1) * x) <= TOL
    dxr, dkr, dw = ops.fftconv_residual_bwd(dy.cuda(), x.cuda(), k.cuda(), omega.cuda())
    assert rel_err(dxr, wdx + omega.view(1, D, 1) * dy) <= TOL and rel_err(dkr, wdk) <= TOL
    assert rel_err(dw, (dy * x).sum(dim=(0, 2))) <= TOL


def test_reference_call_pattern_with_complex128_spectra():
    """fused_ops/fftconv.py:79-106 in double: k_f = rfft(k, 2N) complex128 in,
    (y, x_f) out, backward from (dy, x_f, k_f)."""
    B, D, L = 2, 3, 300
    g = torch.Generator().manual_seed(9)
    x = torch.randn(B, D, L, generator=g, dtype=torch.float64)
    k = torch.randn(D, L, generator=g, dtype=torch.float64) / math.sqrt(L)
    dy = torch.randn(B, D, L, generator=g, dtype=torch.float64)
    N = 1 << (L - 1).bit_length()
    k_f = torch.fft.rfft(k.cuda(), n=2 * N)
    y, x_f = ops.fftconv_fwd(x.cuda(), k_f)
    assert x_f.dtype == torch.complex128 and x_f.shape == (B, D, N + 1)
    assert rel_err(x_f, torch.fft.rfft(x, n=2 * N)) <= TOL
    assert rel_err(y, offt.fftconv_fwd(x, k)) <= TOL
    dx, dk = ops.fftconv_bwd(dy.cuda(), x_f, k_f, torch.float64)
    wdx, wdk = offt.fftconv_bwd(dy, x, k)
    assert rel_err(dx, wdx) <= TOL and rel_err(dk, wdk) <= TOL
