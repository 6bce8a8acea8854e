"""LayerNorm / RMSNorm with stored weight = gamma - 1 against float64
(`torch.nn.functional.layer_norm` and the RMS formula with autograd):
rel err <= 1e-4 float32, <= 2e-2 bfloat16 / float16, outputs and all gradients."""
import pytest
import torch
import torch.nn.functional as F

from conftest import rel_err
from megalodon_amd import extension as ops
from megalodon_amd.fused_ops import layer_norm_plus_one
from megalodon_amd.modules.layer_norm import FusedLayerNorm, FusedRMSNorm

pytestmark = pytest.mark.gpu


def _reference(x, w, b, eps, rms, dy):
    x64 = x.double().requires_grad_(True)
    w64 = None if w is None else w.double().requires_grad_(True)
    b64 = None if b is None else b.double().requires_grad_(True)
    gamma = None if w64 is None else w64 + 1.0
    if rms:
        y = x64 * torch.rsqrt(x64.pow(2).mean(-1, keepdim=True) + eps)
        y = y if gamma is None else y * gamma
    else:
        y = F.layer_norm(x64, x64.shape[-1:], gamma, b64, eps)
    y.backward(dy.double())
    return y.detach(), x64.grad, None if w64 is None else w64.grad, None if b64 is None else b64.grad


@pytest.mark.parametrize("dtype,tol", [(torch.bfloat16, 2e-2), (torch.float16, 2e-2), (torch.float32, 1e-4)])
@pytest.mark.parametrize("rms", [False, True])
@pytest.mark.parametrize("shape,affine", [
    ((2, 70, 4096), True),     # the block's model width: one row per wavefront, 8 chunks per lane
    ((3, 33, 2, 256), False),  # per-head norm of z: two rows per wavefront, no parameters
    ((5, 128), True),          # four rows per wavefront
    ((2, 9, 1024), True),
    ((4, 25, 200), True),      # no register-resident variant: element-wise kernels
    ((1300, 64), True),        # more rows than one pass of the grid... and short rows
    ((1, 1, 512), False),
])
def test_norm_matches_float64(shape, affine, rms, dtype, tol):
    g = torch.Generator().manual_seed(shape[-1] + len(shape))
    D = shape[-1]
    x = (torch.randn(*shape, generator=g) * 1.5 + 0.7).to(dtype)
    dy = torch.randn(*shape, generator=g).to(dtype)
    w = (torch.randn(D, generator=g) * 0.3).to(dtype) if affine else None
    b = (torch.randn(D, generator=g) * 0.3).to(dtype) if affine and not rms else None
    xg = x.cuda().requires_grad_(True)
    wg = None if w is None else w.cuda().requires_grad_(True)
    bg = None if b is None else b.cuda().requires_grad_(True)
    y = layer_norm_plus_one(xg, wg, bg, 1e-5, rms)
    y.backward(dy.cuda())
    wy, wdx, wdw, wdb = _reference(x, w, b, 1e-5, rms, dy)
    assert y.dtype == dtype and y.shape == x.shape
    assert rel_err(y, wy) <= tol and rel_err(xg.grad, wdx) <= tol
    if affine:
        # sums over up to 1300 rows of 16-bit products, rounded to the parameter's type
        assert rel_err(wg.grad, wdw) <= tol
        if not rms:
            assert rel_err(bg.grad, wdb) <= tol


def test_modules_use_the_kernels_and_keep_the_stored_weight_convention():
    torch.manual_seed(0)
    ln, rn, zn = FusedLayerNorm(512).cuda().bfloat16(), FusedRMSNorm(512).cuda().bfloat16(), \
        FusedRMSNorm(64, elementwise_affine=False).cuda()
    x = torch.randn(4, 10, 512, device="cuda", dtype=torch.bfloat16)
    # zero stored weight = plain normalisation
    assert rel_err(ln(x), F.layer_norm(x.double(), (512,))) <= 2e-2
    assert rel_err(rn(x), x.double() * torch.rsqrt(x.double().pow(2).mean(-1, keepdim=True) + 1e-5)) <= 2e-2
    with torch.no_grad():
        ln.weight.fill_(1.0)
        ln.bias.fill_(0.5)
    assert rel_err(ln(x), 2 * F.layer_norm(x.double(), (512,)) + 0.5) <= 2e-2
    z = torch.randn(2, 5, 8, 64, device="cuda", dtype=torch.bfloat16)
    assert rel_err(zn(z), z.double() * torch.rsqrt(z.double().pow(2).mean(-1, keepdim=True) + 1e-5)) <= 2e-2
    # a float32 module takes the same entry point (element-wise kernels)
    ln32 = FusedLayerNorm(512).cuda()
    assert rel_err(ln32(x.float()), F.layer_norm(x.double(), (512,))) <= 1e-4


def test_saved_statistics_and_argument_checks():
    x = torch.randn(6, 256, device="cuda", dtype=torch.bfloat16)
    y, mean, rstd = ops.layer_norm_fwd(x, None, None, 1e-5, False)
    assert rel_err(mean, x.double().mean(-1)) <= 1e-5
    assert rel_err(rstd, torch.rsqrt(x.double().var(-1, unbiased=False) + 1e-5)) <= 1e-5
    y, mean, rstd = ops.layer_norm_fwd(x, None, None, 1e-5, True)
    assert mean is None and rel_err(rstd, torch.rsqrt(x.double().pow(2).mean(-1) + 1e-5)) <= 1e-5
    with pytest.raises(RuntimeError, match="weight must be"):
        ops.layer_norm_fwd(x, torch.zeros(255, device="cuda", dtype=torch.bfloat16), None, 1e-5, False)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.layer_norm_fwd(x.cpu(), None, None, 1e-5, False)
    e = torch.empty(0, 256, device="cuda", dtype=torch.bfloat16)
    assert ops.layer_norm_fwd(e, None, None, 1e-5, False)[0].shape == (0, 256)


def test_full_size_rows_are_independent():
    # config-4 activation (32768 rows of 4096): every row depends on itself only
    x = torch.randn(32768, 4096, device="cuda").bfloat16()
    w = (torch.randn(4096, device="cuda") * 0.1).bfloat16()
    b = (torch.randn(4096, device="cuda") * 0.1).bfloat16()
    dy = torch.randn(32768, 4096, device="cuda").bfloat16()
    for rms in (False, True):
        y, mean, rstd = ops.layer_norm_fwd(x, w, None if rms else b, 1e-5, rms)
        dx, dw, db = ops.layer_norm_bwd(dy, x, w, mean, rstd, rms, not rms)
        idx = torch.tensor([0, 1, 4095, 17000, 32767], device="cuda")
        ys, ms, rs = ops.layer_norm_fwd(x[idx], w, None if rms else b, 1e-5, rms)
        dxs, _, _ = ops.layer_norm_bwd(dy[idx], x[idx], w, ms, rs, rms, not rms)
        assert torch.equal(y[idx], ys) and torch.equal(dx[idx], dxs)
        wy, wdx, wdw, wdb = _reference(x[idx].cpu(), w.cpu(), None if rms else b.cpu(), 1e-5, rms, dy[idx].cpu())
        assert rel_err(ys, wy) <= 2e-2 and rel_err(dxs, wdx) <= 2e-2
        # parameter gradients are sums over all rows: linear in dy
        dx2, dw2, db2 = ops.layer_norm_bwd(dy * 2, x, w, mean, rstd, rms, not rms)
        assert rel_err(dw2, dw.double() * 2) <= 2e-2
        xh = (x.double() - (0 if rms else mean.double()[:, None])) * rstd.double()[:, None]
        assert rel_err(dw, (dy.double() * xh).sum(0)) <= 2e-2
        if not rms:
            assert rel_err(db, dy.double().sum(0)) <= 2e-2


@pytest.mark.parametrize("D,rms", [(4096, False), (8192, False), (8192, True), (10000, True)])
def test_float32_rows_wider_than_one_stripe_per_wave(D, rms):
    """float32 rows take the element-wise kernels, whose parameter-gradient
    stripes share 64 KB of LDS: 4, 2 or 1 working waves per workgroup."""
    g = torch.Generator().manual_seed(D)
    x = torch.randn(3, 11, D, generator=g)
    dy = torch.randn(3, 11, D, generator=g)
    w = torch.randn(D, generator=g) * 0.2
    b = None if rms else torch.randn(D, generator=g) * 0.2
    xg, wg = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    bg = None if b is None else b.cuda().requires_grad_(True)
    y = layer_norm_plus_one(xg, wg, bg, 1e-5, rms)
    y.backward(dy.cuda())
    wy, wdx, wdw, wdb = _reference(x, w, b, 1e-5, rms, dy)
    assert rel_err(y, wy) <= 1e-4 and rel_err(xg.grad, wdx) <= 1e-4 and rel_err(wg.grad, wdw) <= 1e-4
    if not rms:
        assert rel_err(bg.grad, wdb) <= 1e-4


def test_parameter_gradients_that_do_not_fit_are_refused():
    x = torch.randn(4, 10000, device="cuda")
    w = torch.zeros(10000, device="cuda")
    y, mean, rstd = ops.layer_norm_fwd(x, w, w, 1e-5, False)
    with pytest.raises(RuntimeError, match="do not fit"):
        ops.layer_norm_bwd(torch.ones_like(x), x, w, mean, rstd, False, True)
    dx, dw, db = ops.layer_norm_bwd(torch.ones_like(x), x, None, mean, rstd, False, False)   # no parameters: fine
    assert dw is None and db is None and torch.isfinite(dx).all()
