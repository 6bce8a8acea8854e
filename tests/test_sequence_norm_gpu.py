"""Whole-sequence (group) normalisation through the C ABI against the float64
oracle on the same (rounded) inputs: rel err <= 1e-4 for float32, <= 2e-2 for
bfloat16 / float16, forward outputs, saved statistics and every gradient."""
import pytest
import torch

from conftest import rel_err
from megalodon_amd import extension as ops
from oracle import sequence_norm as sn

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2, torch.float16: 2e-2}


def _case(B, L, H, dtype, seed, mask, length_last):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(B, L, H, generator=g) * 1.5 + torch.randn(H, generator=g)).to(dtype)
    dy = torch.randn(B, L, H, generator=g).to(dtype)
    gamma = (1.0 + 0.3 * torch.randn(H, generator=g)).to(dtype)
    beta = (0.2 * torch.randn(H, generator=g)).to(dtype)
    if mask == "holes":
        m = torch.rand(B, L, generator=g) < 0.3
    elif mask == "trailing":
        lens = torch.randint(1, L + 1, (B,), generator=g)
        m = torch.arange(L).unsqueeze(0) >= lens.unsqueeze(1)
    else:
        m = None
    if length_last:
        x, dy = x.transpose(1, 2).contiguous(), dy.transpose(1, 2).contiguous()
    return x, dy, gamma, beta, m


def _check(B, L, H, G, dtype, seed, mask, length_last):
    x, dy, gamma, beta, m = _case(B, L, H, dtype, seed, mask, length_last)
    tol = TOL[dtype]
    dev = lambda t: None if t is None else t.cuda()
    y, count, mean, rstd = ops.group_sequence_norm_fwd(dev(x), dev(gamma), dev(beta), dev(m), G, 1e-5, length_last)
    wy, wcount, wmean, wrstd = sn.group_sequence_norm_fwd(x, gamma, beta, m, G, 1e-5, length_last)
    assert y.dtype == dtype and y.shape == x.shape and mean.dtype == torch.float32
    assert torch.equal(count.cpu(), wcount)
    assert rel_err(mean, wmean) <= 1e-4 and rel_err(rstd, wrstd) <= 1e-4
    assert rel_err(y, wy) <= tol
    dx, dg, db = ops.group_sequence_norm_bwd(dev(dy), dev(x), count, mean, rstd, dev(gamma), dev(m), G, length_last)
    wdx, wdg, wdb = sn.group_sequence_norm_bwd(dy, x, wcount, wmean, wrstd, gamma, m, G, length_last)
    assert dx.dtype == dtype and dg.dtype == dtype and dg.shape == (H,)
    assert rel_err(dx, wdx) <= tol
    assert rel_err(dg, wdg) <= tol
    assert rel_err(db, wdb) <= tol
    if m is not None and m.any():
        mb = m.unsqueeze(1).expand_as(x) if length_last else m.unsqueeze(2).expand_as(x)
        assert y.cpu()[mb].abs().max() == 0 and dx.cpu()[mb].abs().max() == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("length_last", [False, True])
@pytest.mark.parametrize("shape", [
    (2, 300, 64, 8),     # vector path, several tiles (features last)
    (3, 77, 12, 3),      # scalar path: D = 4
    (2, 130, 10, 10),    # per-feature operator, ragged tile
    (1, 4104, 16, 2),    # three tiles of the length-last layout, L % 8 == 0
    (2, 2049, 6, 1),     # one group over everything, odd length
    (1, 1, 8, 2),        # single step
    (2, 200, 48, 16),    # 16-byte loads that straddle groups of D = 3
    (2, 260, 32, 32),    # per-feature operator on the 16-byte path
])
def test_matches_oracle(shape, length_last, dtype):
    B, L, H, G = shape
    for mask in (None, "holes", "trailing"):
        _check(B, L, H, G, dtype, L + H, mask, length_last)


def test_per_feature_operator_and_large_offset():
    """sequence_norm_fwd/bwd = one group per feature; a mean far from zero
    checks that the variance does not come from E[x^2] - E[x]^2."""
    B, L, H = 2, 1000, 32
    g = torch.Generator().manual_seed(0)
    x = 100.0 + 0.1 * torch.randn(B, L, H, generator=g)
    dy = torch.randn(B, L, H, generator=g)
    gamma, beta = torch.ones(H), torch.zeros(H)
    y, count, mean, rstd = ops.sequence_norm_fwd(x.cuda(), gamma.cuda(), beta.cuda(), None, 1e-5)
    wy, wcount, wmean, wrstd = sn.group_sequence_norm_fwd(x, gamma, beta, None, H, 1e-5)
    assert mean.shape == (B, H)
    assert rel_err(rstd, wrstd) <= 1e-4 and rel_err(y, wy) <= 1e-3  # x - mean loses 3 digits at |x| = 1000 sigma
    dx, dg, db = ops.sequence_norm_bwd(dy.cuda(), x.cuda(), count, mean, rstd, gamma.cuda(), None)
    wdx, wdg, wdb = sn.group_sequence_norm_bwd(dy, x, wcount, wmean, wrstd, gamma, None, H)
    assert rel_err(dx, wdx) <= 1e-3 and rel_err(dg, wdg) <= 1e-3 and rel_err(db, wdb) <= 1e-4


def test_hot_path_size_properties():
    """(B, L, H) = (2, 8192, 4096) bf16, 64 groups: the output's per-group
    statistics over the sequence are 0 and 1 when gamma = 1, beta = 0, and the
    forward is invariant to a shift and positive scaling of the input."""
    B, L, H, G = 2, 8192, 4096, 64
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn(B, L, H, generator=g, device="cuda").bfloat16()
    one, zero = torch.ones(H, device="cuda").bfloat16(), torch.zeros(H, device="cuda").bfloat16()
    y, count, mean, rstd = ops.group_sequence_norm_fwd(x, one, zero, None, G, 1e-5)
    assert (count == L).all()
    yg = y.float().view(B, L, G, H // G)
    assert yg.mean((1, 3)).abs().max() < 2e-3
    assert (yg.var((1, 3), unbiased=False) - 1).abs().max() < 5e-3
    x2 = (x.float() * 4.0 + 8.0).bfloat16()  # exact in bf16 up to the shift's rounding
    y2, *_ = ops.group_sequence_norm_fwd(x2, one, zero, None, G, 1e-5)
    assert rel_err(y2, y) <= 2e-2


def test_fully_masked_and_empty():
    B, L, H, G = 2, 40, 16, 4
    x, dy, gamma, beta, m = _case(B, L, H, torch.float32, 3, "holes", False)
    m[1] = True
    y, count, mean, rstd = ops.group_sequence_norm_fwd(x.cuda(), gamma.cuda(), beta.cuda(), m.cuda(), G, 1e-5)
    assert count[1] == 0 and y[1].abs().max() == 0 and mean[1].abs().max() == 0
    dx, dg, db = ops.group_sequence_norm_bwd(dy.cuda(), x.cuda(), count, mean, rstd, gamma.cuda(), m.cuda(), G)
    wy, wc, wm, wr = sn.group_sequence_norm_fwd(x, gamma, beta, m, G, 1e-5)
    wdx, wdg, wdb = sn.group_sequence_norm_bwd(dy, x, wc, wm, wr, gamma, m, G)
    assert dx[1].abs().max() == 0 and rel_err(dx, wdx) <= 1e-4 and rel_err(dg, wdg) <= 1e-4
    # no steps at all / no sequences at all
    e = torch.zeros(2, 0, H, device="cuda")
    y, count, mean, rstd = ops.group_sequence_norm_fwd(e, gamma.cuda(), beta.cuda(), None, G, 1e-5)
    assert y.shape == (2, 0, H) and (count == 0).all() and (mean == 0).all()
    dx, dg, db = ops.group_sequence_norm_bwd(e, e, count, mean, rstd, gamma.cuda(), None, G)
    assert (dg == 0).all() and (db == 0).all()
    e = torch.zeros(0, 5, H, device="cuda")
    y, count, mean, rstd = ops.group_sequence_norm_fwd(e, gamma.cuda(), beta.cuda(), None, G, 1e-5)
    dx, dg, db = ops.group_sequence_norm_bwd(e, e, count, mean, rstd, gamma.cuda(), None, G)
    assert y.shape == (0, 5, H) and (dg == 0).all() and (db == 0).all()


def test_argument_errors():
    x = torch.zeros(2, 8, 12, device="cuda")
    w = torch.ones(12, device="cuda")
    with pytest.raises(RuntimeError, match="num_groups"):
        ops.group_sequence_norm_fwd(x, w, w, None, 5, 1e-5)
    with pytest.raises(RuntimeError, match="padding_mask"):
        ops.group_sequence_norm_fwd(x, w, w, torch.zeros(2, 7, dtype=torch.bool, device="cuda"), 3, 1e-5)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.group_sequence_norm_fwd(x.cpu(), w.cpu(), w.cpu(), None, 3, 1e-5)


@pytest.mark.parametrize("length_last", [False, True])
@pytest.mark.parametrize("groups", [4, None])
def test_autograd_wrapper_matches_oracle_autograd(groups, length_last):
    """fused_ops.sequence_norm through torch.autograd against autograd over the
    float64 oracle forward: y and the gradients of x, gamma and beta."""
    from megalodon_amd.fused_ops import sequence_norm
    B, L, H = 2, 300, 64
    x, dy, gamma, beta, m = _case(B, L, H, torch.float32, 5, "holes", length_last)
    cx, cg, cb = (t.cuda().requires_grad_(True) for t in (x, gamma, beta))
    y = sequence_norm(cx, cg, cb, m.cuda(), groups, 1e-5, length_last)
    y.backward(dy.cuda())
    x64, g64, b64 = (t.double().requires_grad_(True) for t in (x, gamma, beta))
    want, *_ = sn.group_sequence_norm_fwd(x64, g64, b64, m, H if groups is None else groups, 1e-5, length_last)
    want.backward(dy.double())
    assert rel_err(y, want.detach()) <= 1e-4
    for got, ref in ((cx.grad, x64.grad), (cg.grad, g64.grad), (cb.grad, b64.grad)):
        assert rel_err(got, ref) <= 1e-4
