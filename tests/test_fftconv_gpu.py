"""Parity of the HIP causal FFT convolution with the float64 oracle.
Tolerances: rel err (max|a-b|/max|b|) <= 1e-4 for every float32 tensor (rows of
float32 input, and dk / d omega whatever the input dtype), <= 2e-2 for
bfloat16 / float16 tensors.  The default engine computes in float32; the
opt-in matrix-core engine (MEGA_FFTCONV_F16_STAGES=1, fp16 between its DFT
stages) is tested beside it and holds dk to 5e-3 only, which is why it is not
the default."""
import pytest
import torch

from conftest import rel_err
from megalodon_amd import extension as ops
from megalodon_amd import synthetic
from megalodon_amd.fused_ops import ema_parameters, fftconv as fftconv_op, fftconv_residual
from oracle import cema, fftconv

pytestmark = pytest.mark.gpu
TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2, torch.float16: 2e-2}
F16_STAGE_DK = 5e-3   # float32 outputs of the opt-in fp16-stage engine (measured 1.1e-3)


@pytest.fixture(params=["fp32", "f16_stages"])
def engine(request, monkeypatch):
    """Both convolution engines for 16-bit rows: the default float32 one and the
    opt-in matrix-core one (the library reads the variable per call)."""
    if request.param == "f16_stages":
        monkeypatch.setenv("MEGA_FFTCONV_F16_STAGES", "1")
    else:
        monkeypatch.delenv("MEGA_FFTCONV_F16_STAGES", raising=False)
    return request.param


@pytest.fixture
def f16_stages(monkeypatch):
    monkeypatch.setenv("MEGA_FFTCONV_F16_STAGES", "1")


def f32_tol(engine, dtype):
    """Bar for a float32 output computed from rows of `dtype`."""
    return F16_STAGE_DK if (engine == "f16_stages" and dtype != torch.float32) else 1e-4

SHAPES = [
    (1, 3, 1), (2, 3, 31), (2, 5, 50), (1, 4, 2048), (2, 3, 1000),     # direct (time-domain) kernel
    (1, 3, 2049), (2, 2, 4096), (1, 3, 4097), (2, 2, 6001),            # M = 2048, 4096
    (1, 3, 8192), (1, 2, 8193), (2, 2, 16384), (1, 2, 12345),          # M = 4096, 8192
    (1, 3, 16385), (2, 3, 32768), (1, 2, 32767), (1, 2, 20001),        # M = 16384 (even and odd L)
    # several 16-bit rows per workgroup pass (8, 4 or 2), full and ragged last passes
    (3, 5, 2056), (1, 16, 4096), (2, 9, 6000), (1, 11, 8192), (2, 5, 12344), (3, 3, 16384),
]


def _data(B, D, L, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, D, L, generator=g).to(dtype)
    k = torch.randn(D, L, generator=g) * (0.97 ** torch.arange(L, dtype=torch.float32))
    dy = torch.randn(B, D, L, generator=g).to(dtype)
    return x, k, dy


@pytest.mark.parametrize("B,D,L", SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_fwd_matches_oracle(B, D, L, dtype, engine):
    x, k, _ = _data(B, D, L, dtype, 31 * L + B)
    y = ops.fftconv_fwd(x.cuda(), k.cuda())
    assert y.dtype == dtype and y.shape == x.shape
    want = fftconv.fftconv_fwd(x, k)
    assert rel_err(y, want) <= TOL[dtype]


@pytest.mark.parametrize("B,D,L", SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_bwd_matches_oracle(B, D, L, dtype, engine):
    x, k, dy = _data(B, D, L, dtype, 17 * L + B)
    dx, dk = ops.fftconv_bwd(dy.cuda(), x.cuda(), k.cuda(), torch.float32)
    assert dx.dtype == dtype and dk.dtype == torch.float32 and dk.shape == k.shape
    wdx, wdk = fftconv.fftconv_bwd(dy, x, k)
    assert rel_err(dx, wdx) <= TOL[dtype]
    assert rel_err(dk, wdk) <= f32_tol(engine, dtype)


RES_SHAPES = [(2, 3, 50), (1, 4, 2048), (2, 3, 4097), (1, 3, 8192), (2, 2, 12345), (2, 3, 32768), (1, 2, 32767),
              (2, 9, 3000), (1, 7, 8200), (3, 3, 16384)]


@pytest.mark.parametrize("B,D,L", RES_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_residual_variant_matches_oracle(B, D, L, dtype, engine):
    """y = fftconv(x, k) + omega x and its three gradients; the expected values
    are the float64 oracle convolution plus the skip term written out."""
    x, k, dy = _data(B, D, L, dtype, 7 * L + B)
    omega = torch.randn(D, 1, generator=torch.Generator().manual_seed(L)) * 0.5
    y = ops.fftconv_residual_fwd(x.cuda(), k.cuda(), omega.cuda())
    assert y.dtype == dtype and y.shape == x.shape
    w64 = omega.double().view(1, D, 1)
    want = fftconv.fftconv_fwd(x, k).double() + w64 * x.double()
    assert rel_err(y, want) <= TOL[dtype]
    dx, dk, dw = ops.fftconv_residual_bwd(dy.cuda(), x.cuda(), k.cuda(), omega.cuda())
    wdx, wdk = fftconv.fftconv_bwd(dy, x, k)
    assert rel_err(dx, wdx.double() + w64 * dy.double()) <= TOL[dtype]
    assert rel_err(dk, wdk) <= f32_tol(engine, dtype)
    assert dw.shape == (D,) and rel_err(dw, (dy.double() * x.double()).sum(dim=(0, 2))) <= f32_tol(engine, dtype)


@pytest.mark.parametrize("B,D,L", [(1, 3, 32768), (2, 2, 20000), (2, 4, 16384), (1, 8, 8192), (3, 16, 4096),
                                   (2, 8, 2056), (1, 4, 12344)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_saved_spectrum_pair_matches_oracle(B, D, L, dtype, f16_stages):
    """Forward that keeps the spectra of x and k, backward from dy and the two
    buffers alone: same values and gradients as the float64 oracle."""
    x, k, dy = _data(B, D, L, dtype, 13 * L + B)
    omega = torch.randn(D, 1, generator=torch.Generator().manual_seed(L)) * 0.5
    assert ops.fftconv_spectrum_bytes(dtype, B, D, L) > 0
    y, sx, sk = ops.fftconv_residual_fwd_saving(x.cuda(), k.cuda(), omega.cuda())
    w64 = omega.double().view(1, D, 1)
    assert rel_err(y, fftconv.fftconv_fwd(x, k).double() + w64 * x.double()) <= TOL[dtype]
    dx, dk, dw = ops.fftconv_residual_bwd_saved(dy.cuda(), sx, sk, omega.cuda())
    wdx, wdk = fftconv.fftconv_bwd(dy, x, k)
    assert rel_err(dx, wdx.double() + w64 * dy.double()) <= TOL[dtype]
    assert rel_err(dk, wdk) <= F16_STAGE_DK
    assert rel_err(dw, (dy.double() * x.double()).sum(dim=(0, 2))) <= F16_STAGE_DK
    # the recomputing pair gives the same forward bits
    assert torch.equal(y, ops.fftconv_residual_fwd(x.cuda(), k.cuda(), omega.cuda()))


@pytest.mark.parametrize("B,D,L", [(3, 256, 20000), (2, 1024, 4096), (2, 130, 32768), (4, 520, 9000)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_batch_walking_forward_matches_oracle(B, D, L, dtype, f16_stages):
    """B > 1 with at least half as many channel groups as compute units: the
    forward that transforms k once per channel group and walks the batch, with
    and without kept spectra, and the backward from those spectra (the
    spectrum of k is kept once per channel)."""
    x, k, dy = _data(B, D, L, dtype, 17 * L + B)
    omega = torch.randn(D, 1, generator=torch.Generator().manual_seed(L)) * 0.5
    w64 = omega.double().view(1, D, 1)
    want = fftconv.fftconv_fwd(x, k).double()
    y0 = ops.fftconv_fwd(x.cuda(), k.cuda())
    assert rel_err(y0, want) <= TOL[dtype]
    y1 = ops.fftconv_residual_fwd(x.cuda(), k.cuda(), omega.cuda())
    assert rel_err(y1, want + w64 * x.double()) <= TOL[dtype]
    if ops.fftconv_spectrum_bytes(dtype, B, D, L) == 0:
        return
    y, sx, sk = ops.fftconv_residual_fwd_saving(x.cuda(), k.cuda(), omega.cuda())
    assert torch.equal(y, y1)
    assert sk.numel() == ops.fftconv_spectrum_bytes(dtype, 1, D, L) and sx.numel() == B * sk.numel()
    dx, dk, dw = ops.fftconv_residual_bwd_saved(dy.cuda(), sx, sk, omega.cuda())
    wdx, wdk = fftconv.fftconv_bwd(dy, x, k)
    assert rel_err(dx, wdx.double() + w64 * dy.double()) <= TOL[dtype]
    assert rel_err(dk, wdk) <= F16_STAGE_DK
    assert rel_err(dw, (dy.double() * x.double()).sum(dim=(0, 2))) <= F16_STAGE_DK
    # every batch entry on its own (B = 1: the kernel that transforms k per row) gives the same rows
    for b in range(B):
        assert torch.equal(ops.fftconv_residual_fwd(x[b:b + 1].cuda(), k.cuda(), omega.cuda())[0], y1[b])


def test_saved_spectrum_pair_at_full_row_count_agrees_with_recomputing_pair(f16_stages):
    """Config-1 rows (L = 32768, bf16) over 512 channels and two batch entries:
    the backward from kept spectra and the backward that re-transforms x and k
    see the same fp16 spectra, so they agree far inside the bfloat16 bar."""
    B, D, L = 2, 512, 32768
    g = torch.Generator().manual_seed(91)
    x = torch.randn(B, D, L, generator=g).bfloat16().cuda()
    dy = torch.randn(B, D, L, generator=g).bfloat16().cuda()
    k = (torch.randn(D, L, generator=g) * (0.9995 ** torch.arange(L, dtype=torch.float32))).cuda()
    omega = torch.randn(D, generator=g).cuda()
    y, sx, sk = ops.fftconv_residual_fwd_saving(x, k, omega)
    assert torch.equal(y, ops.fftconv_residual_fwd(x, k, omega))
    dx, dk, dw = ops.fftconv_residual_bwd_saved(dy, sx, sk, omega)
    rdx, rdk, rdw = ops.fftconv_residual_bwd(dy, x, k, omega)
    assert rel_err(dx, rdx) <= 4e-3 and rel_err(dk, rdk) <= 1e-3 and rel_err(dw, rdw) <= 1e-3


def test_saved_spectrum_path_is_off_without_the_switch(monkeypatch):
    monkeypatch.delenv("MEGA_FFTCONV_F16_STAGES", raising=False)
    assert ops.fftconv_spectrum_bytes(torch.bfloat16, 1, 8, 4096) == 0


def test_saved_spectrum_path_is_refused_outside_its_shapes(f16_stages):
    assert ops.fftconv_spectrum_bytes(torch.bfloat16, 1, 8, 4096) > 0
    assert ops.fftconv_spectrum_bytes(torch.float32, 1, 8, 4096) == 0
    assert ops.fftconv_spectrum_bytes(torch.bfloat16, 1, 8, 2048) == 0
    assert ops.fftconv_spectrum_bytes(torch.bfloat16, 1, 3, 4096) == 0   # 8 rows per pass, D = 3
    assert ops.fftconv_spectrum_bytes(torch.bfloat16, 1, 8, 4097) == 0
    x = torch.zeros(1, 3, 4096, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="saved-spectrum"):
        ops.fftconv_residual_fwd_saving(x, torch.zeros(3, 4096, device="cuda"), torch.zeros(3, device="cuda"))


def test_residual_autograd_function_16bit(engine):
    """bf16 rows through the autograd node: kept (x, k) on the default engine,
    kept spectra on the opt-in one."""
    x, k, dy = _data(2, 8, 6000, torch.bfloat16, 3)
    omega = torch.randn(8, 1)
    xg, kg, wg = (t.cuda().requires_grad_() for t in (x, k, omega))
    fftconv_residual(xg, kg, wg).backward(dy.cuda())
    wdx, wdk = fftconv.fftconv_bwd(dy, x, k)
    assert rel_err(xg.grad, wdx.double() + omega.double().view(1, 8, 1) * dy.double()) <= 2e-2
    assert rel_err(kg.grad, wdk) <= f32_tol(engine, torch.bfloat16)
    assert rel_err(wg.grad.view(-1), (dy.double() * x.double()).sum(dim=(0, 2))) <= f32_tol(engine, torch.bfloat16)


def test_residual_autograd_function():
    x, k, dy = _data(2, 3, 3000, torch.float32, 3)
    omega = torch.randn(3, 1)
    xg, kg, wg = (t.cuda().requires_grad_() for t in (x, k, omega))
    fftconv_residual(xg, kg, wg).backward(dy.cuda())
    xr, kr, wr = (t.cuda().requires_grad_() for t in (x, k, omega))
    (fftconv_op(xr, kr) + xr * wr).backward(dy.cuda())
    assert rel_err(xg.grad, xr.grad) <= 1e-4 and rel_err(kg.grad, kr.grad) <= 1e-4
    assert wg.grad.shape == omega.shape and rel_err(wg.grad, wr.grad) <= 1e-4


@pytest.mark.parametrize("B,D,L", [(2, 3, 5000), (1, 5, 2400), (2, 3, 10000), (1, 2, 30000)])
def test_float16_rows(B, D, L, engine):
    x, k, dy = _data(B, D, L, torch.float16, 5)
    y = ops.fftconv_fwd(x.cuda(), k.cuda())
    assert rel_err(y, fftconv.fftconv_fwd(x, k)) <= TOL[torch.float16]
    dx, dk = ops.fftconv_bwd(dy.cuda(), x.cuda(), k.cuda(), torch.float32)
    wdx, wdk = fftconv.fftconv_bwd(dy, x, k)
    assert rel_err(dx, wdx) <= TOL[torch.float16] and rel_err(dk, wdk) <= f32_tol(engine, torch.float16)


def test_rows_of_a_pass_do_not_mix(f16_stages):
    """Short 16-bit rows share a workgroup pass: a row of zeros between busy
    rows stays exactly zero, and every row equals its single-row result."""
    B, D, L = 1, 8, 4096
    x, k, _ = _data(B, D, L, torch.bfloat16, 11)
    x[:, 3] = 0
    y = ops.fftconv_fwd(x.cuda(), k.cuda())
    assert y[:, 3].abs().max().item() == 0.0
    for d in (0, 5):
        yd = ops.fftconv_fwd(x[:, d:d + 1].contiguous().cuda(), k[d:d + 1].contiguous().cuda())
        assert torch.equal(yd[:, 0], y[:, d])


def test_config0_cema_forward_fp32():
    """BASELINE config 0: CEMA forward fp32, B=1, L=2048, D=1024, ndim=16."""
    D, N, L = 1024, 16, 2048
    prm = synthetic.cema_params(D, N, 1000)
    x = synthetic.cema_inputs(1, D, L, 1000)["x"]
    k, _ = ema_parameters(prm["p"].cuda(), prm["q"].cuda(), prm["gamma"].cuda(), None, L)
    out = fftconv_op(x.cuda(), k) + x.cuda() * prm["omega"].cuda()
    kk = cema.ema_weight_fwd(prm["p"], prm["q"].log(), prm["gamma"], L)
    want = fftconv.fftconv_fwd(x, kk) + x.double() * prm["omega"].double()
    assert rel_err(out, want) <= 1e-4


def test_config1_rows_bf16_fwd_bwd_with_ema_kernel(engine):
    """BASELINE config 1 row shape (L=32768, ndim=16, x bf16), a slice of the channels."""
    D, N, L = 48, 16, 32768
    prm = synthetic.cema_params(D, N, 1001)
    io = synthetic.cema_inputs(1, D, L, 1001, torch.bfloat16)
    kk = cema.ema_weight_fwd(prm["p"], prm["q"].log(), prm["gamma"], L)
    k = kk.float()
    y = ops.fftconv_fwd(io["x"].cuda(), k.cuda())
    assert rel_err(y, fftconv.fftconv_fwd(io["x"], k)) <= 2e-2
    dx, dk = ops.fftconv_bwd(io["dy"].cuda(), io["x"].cuda(), k.cuda(), torch.float32)
    wdx, wdk = fftconv.fftconv_bwd(io["dy"], io["x"], k)
    assert rel_err(dx, wdx) <= 2e-2
    assert rel_err(dk, wdk) <= f32_tol(engine, torch.bfloat16)


def test_full_size_linearity_and_shift_properties():
    """Size-independent checks at the full benchmark shape of one launch:
    linearity in x and the unit-impulse identity conv(x, delta) = x."""
    B, D, L = 1, 512, 32768
    g = torch.Generator().manual_seed(77)
    x1 = torch.randn(B, D, L, generator=g).cuda()
    x2 = torch.randn(B, D, L, generator=g).cuda()
    k = (torch.randn(D, L, generator=g) * (0.999 ** torch.arange(L, dtype=torch.float32))).cuda()
    y1 = ops.fftconv_fwd(x1, k)
    y2 = ops.fftconv_fwd(x2, k)
    y12 = ops.fftconv_fwd(x1 + 2.0 * x2, k)
    assert rel_err(y12, y1 + 2.0 * y2) <= 1e-4
    delta = torch.zeros(D, L, device="cuda")
    delta[:, 0] = 1.0
    assert rel_err(ops.fftconv_fwd(x1, delta), x1) <= 1e-5
    shift = torch.zeros(D, L, device="cuda")
    shift[:, 5] = 1.0
    ys = ops.fftconv_fwd(x1, shift)
    assert rel_err(ys[..., 5:], x1[..., :-5]) <= 1e-5 and ys[..., :5].abs().max().item() <= 1e-4


def test_autograd_function():
    B, D, L = 2, 4, 3000
    x, k, dy = _data(B, D, L, torch.float32, 9)
    xc = x.cuda().requires_grad_(True)
    kc = k.cuda().requires_grad_(True)
    y = fftconv_op(xc, kc)
    y.backward(dy.cuda())
    wdx, wdk = fftconv.fftconv_bwd(dy, x, k)
    assert rel_err(xc.grad, wdx) <= 1e-4 and rel_err(kc.grad, wdk) <= 1e-4


def test_too_long_rows_fail_loudly_at_the_c_abi():
    from megalodon_amd import _lib
    x = torch.zeros(1, 1, 32776, device="cuda")
    k = torch.zeros(1, 32776, device="cuda")
    y = torch.empty_like(x)
    with pytest.raises(RuntimeError, match="exceeds"):
        _lib.call("mega_fftconv_fwd", _lib.ptr(x), _lib.i32(_lib.dtype_code(x.dtype)), _lib.ptr(k), _lib.i64(1),
                  _lib.i64(1), _lib.i64(32776), _lib.ptr(y), _lib.stream_ptr(x.device))


def _long_data(B, D, L, dtype, seed):
    # a kernel that still weighs 2 % at the end of the row, so every block pair contributes
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, D, L, generator=g).to(dtype)
    k = torch.randn(D, L, generator=g) * torch.exp(-4.0 * torch.arange(L, dtype=torch.float32) / L)
    dy = torch.randn(B, D, L, generator=g).to(dtype)
    return x, k, dy


@pytest.mark.parametrize("B,D,L", [(1, 2, 32769), (2, 3, 40000), (1, 2, 65536), (1, 2, 70001), (1, 1, 131072)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rows_beyond_one_launch_match_oracle(B, D, L, dtype, engine):
    """L > 32768: the host cuts rows into blocks (heads and tails of block
    pairs); forward and backward against the float64 oracle on the whole row."""
    x, k, dy = _long_data(B, D, L, dtype, L + B)
    y = ops.fftconv_fwd(x.cuda(), k.cuda())
    assert y.dtype == dtype and y.shape == x.shape
    assert rel_err(y, fftconv.fftconv_fwd(x, k)) <= TOL[dtype]
    dx, dk = ops.fftconv_bwd(dy.cuda(), x.cuda(), k.cuda(), torch.float32)
    wdx, wdk = fftconv.fftconv_bwd(dy, x, k)
    assert dx.dtype == dtype and dk.shape == k.shape
    assert rel_err(dx, wdx) <= TOL[dtype]
    assert rel_err(dk, wdk) <= f32_tol(engine, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_residual_autograd_function_beyond_one_launch(dtype, engine):
    B, D, L = 2, 3, 50000
    x, k, dy = _long_data(B, D, L, dtype, 77)
    om = torch.randn(D, 1, generator=torch.Generator().manual_seed(5))
    xc, kc, oc = (t.cuda().requires_grad_(True) for t in (x, k, om))
    y = fftconv_residual(xc, kc, oc)
    y.backward(dy.cuda())
    x64, k64, o64 = (t.double().requires_grad_(True) for t in (x, k, om))
    want = fftconv.fftconv_fwd(x64, k64) + x64 * o64
    want.backward(dy.double())
    assert y.dtype == dtype
    assert rel_err(y, want.detach()) <= TOL[dtype]
    assert rel_err(xc.grad, x64.grad) <= TOL[dtype]
    assert rel_err(kc.grad, k64.grad) <= f32_tol(engine, dtype)
    assert rel_err(oc.grad, o64.grad) <= f32_tol(engine, dtype)


def test_cema_layer_at_twice_the_launch_length():
    """MultiHeadComplexEMA forward+backward at L = 65536 (fp32): kernel
    generation, the block-cut convolution and every parameter gradient against
    the float64 closed form + FFT convolution + autograd."""
    from megalodon_amd.modules import MultiHeadComplexEMA
    B, D, N, L = 1, 8, 16, 65536
    torch.manual_seed(3)
    m = MultiHeadComplexEMA(D, N).cuda()
    io = synthetic.cema_inputs(B, D, L, 99)
    x = io["x"].cuda().requires_grad_(True)
    out, _ = m(x, None, False)
    out.backward(io["dy"].cuda())
    pr = {n_: v.detach().cpu().double().requires_grad_(True) for n_, v in m.named_parameters()}
    xo = io["x"].double().requires_grad_(True)
    p, q, g = cema.calc_coeffs(pr["alpha"], pr["delta"], pr["theta"], pr["gamma"], N)
    want = fftconv.fftconv_fwd(xo, cema.ema_weight_fwd(p, q.log(), g, L)) + xo * pr["omega"]
    want.backward(io["dy"].double())
    assert rel_err(out, want.detach()) <= 1e-4
    assert rel_err(x.grad, xo.grad) <= 1e-4
    for n_, prm in m.named_parameters():
        assert rel_err(prm.grad, pr[n_].grad) <= 1e-4, n_


def test_fused_fftconv_pair_has_the_reference_call_pattern():
    """y, a, b = fused_fftconv_fwd(x, k); dx, dk = fused_fftconv_bwd(dy, a, b, k.dtype)."""
    from megalodon_amd.fused_ops import fused_fftconv_bwd, fused_fftconv_fwd
    x, k, dy = _data(2, 3, 5000, torch.float32, 8)
    y, a, b = fused_fftconv_fwd(x.cuda(), k.cuda())
    dx, dk = fused_fftconv_bwd(dy.cuda(), a, b, k.dtype)
    wdx, wdk = fftconv.fftconv_bwd(dy, x, k)
    assert rel_err(y, fftconv.fftconv_fwd(x, k)) <= 1e-4
    assert dk.dtype == k.dtype and rel_err(dx, wdx) <= 1e-4 and rel_err(dk, wdk) <= 1e-4


# The reference's own call pattern (fused_ops/fftconv.py:79-106): the kernel goes
# in as a spectrum, the forward returns (y, x_f), the backward takes the two
# spectra and the kernel's dtype.  Only the import line of that file changes.
def _reference_style_fwd(x, k):
    L = x.size(-1)
    N = L if (L & (L - 1)) == 0 else (1 << L.bit_length())
    if k.dtype in (torch.float32, torch.float64):
        k_f = torch.fft.rfft(k, 2 * N)
    else:
        k_f = ops.rfft(k, False)
    y, x_f = ops.fftconv_fwd(x, k_f)
    return y, x_f, k_f


@pytest.mark.parametrize("B,D,L", [(2, 3, 32), (2, 3, 1000), (1, 4, 4096), (2, 2, 6001), (1, 3, 16384)])
@pytest.mark.parametrize("dtype,k_dtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.float32),
                                           (torch.float16, torch.float16)])
def test_reference_call_pattern_with_spectra(B, D, L, dtype, k_dtype):
    x, k, dy = _data(B, D, L, dtype, 17 * L + D)
    k = k.to(k_dtype)
    N = 1 << (L - 1).bit_length()
    y, x_f, k_f = _reference_style_fwd(x.cuda(), k.cuda())
    assert y.dtype == dtype and y.shape == x.shape
    assert x_f.shape == (B, D, N + 1) and x_f.dtype == torch.complex64 and k_f.shape == (D, N + 1)
    want_xf = torch.fft.rfft(x.double(), n=2 * N)
    assert rel_err(x_f, want_xf) <= 1e-4
    assert rel_err(y, fftconv.fftconv_fwd(x.double(), k.double())) <= TOL[dtype]
    dx, dk = ops.fftconv_bwd(dy.cuda(), x_f, k_f, k_dtype)
    wdx, wdk = fftconv.fftconv_bwd(dy.double(), x.double(), k.double())
    assert dx.dtype == dtype and dk.dtype == k_dtype and dk.shape == (D, L)
    assert rel_err(dx, wdx) <= TOL[dtype]
    assert rel_err(dk, wdk) <= TOL[k_dtype]


def test_spectral_signature_rejects_wrong_bin_count():
    x = torch.zeros(1, 2, 100, device="cuda")
    with pytest.raises(RuntimeError, match="129 bins"):
        ops.fftconv_fwd(x, torch.zeros(2, 101, dtype=torch.complex64, device="cuda"))


def test_prepare_makes_tables_and_scratch_ahead_of_the_first_call():
    """fftconv_prepare(L) does the float32 engine's first-use allocation; the convolution that
    follows on the same stream gives the oracle's result (the call itself then allocates nothing)."""
    B, D, L = 1, 2, 5000
    ops.fftconv_prepare(L)
    x, k, _ = _data(B, D, L, torch.float32, 99)
    y = ops.fftconv_fwd(x.cuda(), k.cuda())
    assert rel_err(y, fftconv.fftconv_fwd(x.double(), k.double())) <= 1e-4
    ops.fftconv_prepare(10 ** 6)          # longer rows are cut into launches of the maximum length: prepared too
