"""Parity of the HIP group TimestepNorm with the float64 oracle (forward values,
statistics and all gradients).  Tolerances: rel err (max|a-b|/max|b|) <= 1e-4
in float32, <= 2e-2 in bfloat16, <= 1e-11 in float64 (the double-precision flavour)."""
import pytest
import torch

from conftest import rel_err
from megalodon_amd import extension as ops
from megalodon_amd import synthetic
from megalodon_amd.modules import TimestepNorm
from oracle import timestep_norm as tn

pytestmark = pytest.mark.gpu
TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2, torch.float64: 1e-11}


def _case(B, L, H, G, seed, dtype, prior=0, mask="trailing"):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(B, L, H, generator=g) + 0.5 * torch.randn(H, generator=g)).to(dtype)
    prev_count = torch.full((B,), prior, dtype=torch.int64)
    prev_mean = (0.3 * torch.randn(B, G, generator=g)).to(dtype)
    prev_var = (0.5 + torch.rand(B, G, generator=g)).to(dtype)
    gamma = (1.0 + 0.1 * torch.randn(H, generator=g)).to(dtype)
    beta = (0.1 * torch.randn(H, generator=g)).to(dtype)
    if mask == "trailing":
        lens = torch.randint(max(1, L // 2), L + 1, (B,), generator=g)
        m = torch.arange(L).unsqueeze(0) >= lens.unsqueeze(1)
    elif mask == "holes":
        m = torch.rand(B, L, generator=g) < 0.3
    else:
        m = None
    dy = torch.randn(B, L, H, generator=g).to(dtype)
    dmean = torch.randn(B, G, generator=g).to(dtype)
    dvar = torch.randn(B, G, generator=g).to(dtype)
    return x, prev_count, prev_mean, prev_var, gamma, beta, m, dy, dmean, dvar


def _cuda(*ts):
    return [None if t is None else t.cuda() for t in ts]


def _run_fwd_bwd(B, L, H, G, dtype, prior, mask, seed, check_stats_everywhere=True, time_last=False):
    x, pc, pm, pv, gamma, beta, m, dy, dmean, dvar = _case(B, L, H, G, seed, dtype, prior, mask)
    eps = 1e-5
    cx, cpc, cpm, cpv, cg, cb, cm = _cuda(x, pc, pm, pv, gamma, beta, m)
    y, count, mean, var, cummean, cumrstd = ops.group_timestep_norm_fwd(cx, cpc, cpm, cpv, cg, cb, cm, G, eps,
                                                                        stats_time_last=time_last)
    wy, wcount, wmean, wvar, wcm, wcr = tn.group_timestep_norm_closed_form_full(x, pc, pm, pv, gamma, beta, m, G, eps)
    if time_last:   # the saved statistics as (B, G, L)
        assert cummean.shape == (B, G, L) and cumrstd.shape == (B, G, L)
        wcm, wcr = wcm.transpose(1, 2), wcr.transpose(1, 2)
    tol = TOL[dtype]
    stat_dtype = torch.float64 if dtype == torch.float64 else torch.float32   # the accumulate type
    assert y.dtype == dtype and cummean.dtype == stat_dtype and count.dtype == torch.int64
    assert torch.equal(count.cpu(), wcount)
    assert rel_err(y, wy) <= tol
    assert rel_err(mean, wmean) <= tol and rel_err(var, wvar) <= tol
    assert rel_err(cummean, wcm) <= min(tol, 1e-4) and rel_err(cumrstd, wcr) <= min(tol, 1e-4)
    # backward consumes the statistics the forward saved
    dx, dpm, dpv, dg, db = ops.group_timestep_norm_bwd(dy.cuda(), dmean.cuda(), dvar.cuda(), cx, cpm, count,
                                                       cummean, cumrstd, cg, cm, G, stats_time_last=time_last)
    want = tn.group_timestep_norm_bwd_autograd(dy, dmean, dvar, x, pc, pm, pv, gamma, beta, m, G, eps)
    for name, a, b_ in zip(["dx", "dprev_mean", "dprev_var", "dgamma", "dbeta"], (dx, dpm, dpv, dg, db), want):
        assert a.dtype == dtype
        assert rel_err(a, b_) <= tol, name


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,L,H,G,prior,mask", [
    (2, 64, 256, 2, 0, None),        # one tile, Dg = 128
    (2, 200, 512, 4, 3, "trailing"), # ragged last tile
    (3, 1000, 384, 3, 5, "holes"),   # interior masked steps, many tiles
    (1, 8192, 256, 2, 0, "trailing"),  # config-2 length: look-back across 128 tiles
    (2, 130, 64, 2, 2, "holes"),     # Dg = 32
    (2, 77, 1024, 2, 1, "trailing"), # Dg = 512 (64 lanes per row in 16-bit)
    (2, 50, 48, 48, 4, "holes"),     # one feature per group: serial path
    (2, 150, 256, 2, 0, "holes"),    # masked steps before the first counted one, no prior
    (2, 33, 36, 1, 0, None),         # one group, Dg not a multiple of the vector width
    (1, 1, 128, 1, 0, None),         # single step
])
def test_fwd_bwd_match_oracle(B, L, H, G, prior, mask, dtype):
    _run_fwd_bwd(B, L, H, G, dtype, prior, mask, seed=B * 1000 + L)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,L,H,G,prior,mask", [
    (2, 200, 512, 4, 3, "trailing"),   # tile-per-wave forward, ragged last tile
    (3, 1000, 384, 3, 5, "holes"),
    (2, 77, 1024, 2, 1, "trailing"),   # workgroup forward kernel (64 lanes per row)
    (2, 50, 48, 48, 4, "holes"),       # serial kernels
    (1, 1, 128, 1, 0, None),
])
def test_statistics_kept_time_last(B, L, H, G, prior, mask, dtype):
    """`stats_time_last`: cummean / cumrstd travel from the forward to the backward as (B, G, L)
    (what the module's autograd node uses); values, statistics and gradients against the oracle as
    in the reference layout, and a layout the backward was not told about is refused."""
    _run_fwd_bwd(B, L, H, G, dtype, prior, mask, seed=B * 1000 + L + 1, time_last=True)
    if L != G:
        x, pc, pm, pv, gamma, beta, m, dy, dmean, dvar = _case(B, L, H, G, 1, dtype, prior, mask)
        cx, cpc, cpm, cpv, cg, cb, cm = _cuda(x, pc, pm, pv, gamma, beta, m)
        _, count, _, _, cmn, crs = ops.group_timestep_norm_fwd(cx, cpc, cpm, cpv, cg, cb, cm, G, 1e-5, stats_time_last=True)
        with pytest.raises(RuntimeError, match="cummean / cumrstd must be"):
            ops.group_timestep_norm_bwd(dy.cuda(), dmean.cuda(), dvar.cuda(), cx, cpm, count, cmn, crs, cg, cm, G)


@pytest.mark.parametrize("B,L,H,G,prior,mask", [
    (2, 200, 512, 4, 3, "trailing"), (3, 300, 384, 3, 5, "holes"), (2, 50, 48, 48, 4, "holes"),
    (2, 33, 36, 1, 0, None), (1, 40, 1200, 2, 0, "holes"),   # the last: groups wider than 256 features
])
def test_float64_tensors(B, L, H, G, prior, mask):
    """The reference instantiates the operator for double (timestep_norm_kernel.cu:1567-1576,
    float64 statistics): forward values, statistics and all gradients to 1e-11."""
    _run_fwd_bwd(B, L, H, G, torch.float64, prior, mask, seed=B * 77 + L)


@pytest.mark.parametrize("offset", [8.0, 40.0])
def test_bf16_forward_with_large_channel_offsets(offset):
    """bfloat16 rows take their moments in one pass (E[x^2] - mean^2 in float32);
    a mean many standard deviations from zero must stay within the bfloat16 bar."""
    B, L, H, G = 2, 300, 512, 4
    x, pc, pm, pv, gamma, beta, m, *_ = _case(B, L, H, G, 7, torch.float32, 0, "holes")
    x = (x + offset).to(torch.bfloat16)
    pm, pv, gamma, beta = (t.to(torch.bfloat16) for t in (pm, pv, gamma, beta))
    y, count, mean, var, cummean, cumrstd = ops.group_timestep_norm_fwd(*_cuda(x, pc, pm, pv, gamma, beta, m), G, 1e-5)
    wy, wcount, wmean, wvar, wcm, wcr = tn.group_timestep_norm_closed_form_full(x, pc, pm, pv, gamma, beta, m, G, 1e-5)
    assert rel_err(y, wy) <= 2e-2 and rel_err(var, wvar) <= 2e-2
    assert rel_err(cummean, wcm) <= 1e-4 and rel_err(cumrstd, wcr) <= 2e-3


@pytest.mark.parametrize("prior", [4, 0])
def test_all_steps_masked_keeps_prior(prior):
    B, L, H, G = 2, 70, 256, 2
    x, pc, pm, pv, gamma, beta, _, *_ = _case(B, L, H, G, 3, torch.float32, prior=prior, mask=None)
    m = torch.ones(B, L, dtype=torch.bool)
    y, count, mean, var, cm, cr = ops.group_timestep_norm_fwd(*_cuda(x, pc, pm, pv, gamma, beta, m), G, 1e-5)
    assert y.abs().max().item() == 0
    assert torch.equal(count.cpu(), pc)
    assert torch.allclose(mean.cpu(), pm) and torch.allclose(var.cpu(), pv)
    assert torch.allclose(cm.cpu(), pm.unsqueeze(1).expand(B, L, G))


def test_config2_shape_slice_bf16():
    """BASELINE config 2 (B=4, L=8192, 32 groups of 128, bf16, trailing padding),
    with D cut to 1024 (8 groups) so the float64 oracle finishes in seconds."""
    B, L, D, G = 4, 8192, 1024, 8
    io = synthetic.timestep_norm_inputs(B, L, D, G, 1002)
    cx = io["x"].cuda()
    y, count, mean, var, cm, cr = ops.group_timestep_norm_fwd(
        cx, io["prev_count"].cuda(), io["prev_mean"].cuda(), io["prev_var"].cuda(), io["gamma"].cuda(),
        io["beta"].cuda(), io["mask"].cuda(), G, 1e-5)
    wy, wcount, wmean, wvar, wcm, wcr = tn.group_timestep_norm_closed_form_full(
        io["x"], io["prev_count"], io["prev_mean"], io["prev_var"], io["gamma"], io["beta"], io["mask"], G, 1e-5)
    assert torch.equal(count.cpu(), wcount)
    assert rel_err(y, wy) <= 2e-2 and rel_err(cm, wcm) <= 1e-4 and rel_err(cr, wcr) <= 1e-4
    dx, dpm, dpv, dg, db = ops.group_timestep_norm_bwd(
        io["dy"].cuda(), io["dmean"].cuda(), io["dvar"].cuda(), cx, io["prev_mean"].cuda(), count, cm, cr,
        io["gamma"].cuda(), io["mask"].cuda(), G)
    want = tn.group_timestep_norm_bwd_autograd(io["dy"], io["dmean"], io["dvar"], io["x"], io["prev_count"],
                                               io["prev_mean"], io["prev_var"], io["gamma"], io["beta"],
                                               io["mask"], G, 1e-5)
    for name, a, b_ in zip(["dx", "dprev_mean", "dprev_var", "dgamma", "dbeta"], (dx, dpm, dpv, dg, db), want):
        assert rel_err(a, b_) <= 2e-2, name


def test_full_config2_properties():
    """Size-independent checks at the full config-2 shape: (i) splitting the
    sequence in two and carrying (count, mean, var) gives the same output as one
    pass; (ii) the per-step output has zero mean / unit variance w.r.t. the
    stored cumulative statistics."""
    B, L, D, G = 4, 8192, 4096, 32
    io = synthetic.timestep_norm_inputs(B, L, D, G, 1002)
    args = [io[k].cuda() for k in ("prev_count", "prev_mean", "prev_var", "gamma", "beta")]
    x, m = io["x"].cuda(), io["mask"].cuda()
    y, count, mean, var, cm, cr = ops.group_timestep_norm_fwd(x, *args, m, G, 1e-5)
    h = L // 2
    y1, c1, m1, v1, _, _ = ops.group_timestep_norm_fwd(x[:, :h].contiguous(), *args, m[:, :h].contiguous(), G, 1e-5)
    y2, c2, m2, v2, _, _ = ops.group_timestep_norm_fwd(x[:, h:].contiguous(), c1, m1, v1, args[3], args[4],
                                                       m[:, h:].contiguous(), G, 1e-5)
    assert torch.equal(c2, count)
    # mean / var are carried in bf16 across the split: compare at bf16 tolerance
    assert rel_err(torch.cat([y1, y2], 1), y) <= 2e-2
    valid = (~m).float()
    assert int(count.sum()) == int(valid.sum())
    xn = (x.float().view(B, L, G, D // G) - cm.unsqueeze(-1)) * cr.unsqueeze(-1)
    z = xn * io["gamma"].cuda().float().view(G, -1) + io["beta"].cuda().float().view(G, -1)
    assert rel_err(y.float().view(B, L, G, -1) , z * valid.view(B, L, 1, 1)) <= 2e-2


def test_module_matches_oracle_with_learned_prior():
    torch.manual_seed(0)
    B, L, D, G = 2, 300, 256, 4
    mod = TimestepNorm(D, G, prior_count=2).cuda()
    with torch.no_grad():
        mod.weight.normal_(0, 0.1)
        mod.bias.normal_(0, 0.1)
        mod.prior_mean.normal_(0, 0.2)
        mod.prior_logv.normal_(0, 0.2)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(B, L, D, generator=g)
    xc = x.cuda().requires_grad_(True)
    y, count, mean, var = mod(xc)
    dy = torch.randn(B, L, D, generator=g)
    (y * dy.cuda()).sum().backward()
    w = {k: v.detach().cpu().double().requires_grad_(True) for k, v in mod.named_parameters()}
    xo = x.double().requires_grad_(True)
    pc = torch.full((B,), 2, dtype=torch.int64)
    yo, mo, vo = tn.group_timestep_norm_closed_form(
        xo, pc, w["prior_mean"].expand(B, -1), w["prior_logv"].exp().expand(B, -1),
        w["weight"] + 1.0, w["bias"], None, G, 1e-5)
    (yo * dy.double()).sum().backward()
    assert rel_err(y, yo) <= 1e-4 and rel_err(xc.grad, xo.grad) <= 1e-4
    for k, v in mod.named_parameters():
        assert rel_err(v.grad, w[k].grad) <= 1e-4, k


def test_dtype_mismatch_is_an_error():
    x, pc, pm, pv, gamma, beta, m, *_ = _case(1, 8, 16, 2, 0, torch.bfloat16)
    with pytest.raises(RuntimeError, match="dtype"):
        ops.group_timestep_norm_fwd(x.cuda(), pc.cuda(), pm.float().cuda(), pv.cuda(), gamma.cuda(), beta.cuda(), None, 2, 1e-5)
    with pytest.raises(RuntimeError, match="divisible"):
        ops.group_timestep_norm_fwd(x.cuda(), pc.cuda(), pm.cuda(), pv.cuda(), gamma.cuda(), beta.cuda(), None, 3, 1e-5)


@pytest.mark.parametrize("mask", [None, "holes"])
def test_non_group_operator(mask):
    """timestep_norm_fwd/bwd (one running mean / variance per feature) equals
    the float64 oracle of the group operator with one feature per group."""
    B, L, H = 2, 90, 24
    x, pc, pm, pv, gamma, beta, m, dy, dmean, dvar = _case(B, L, H, H, 21, torch.float32, 2, mask)
    y, count, mean, var, cm, cr = ops.timestep_norm_fwd(*_cuda(x, pc, pm, pv, gamma, beta, m), 1e-5)
    wy, wcount, wmean, wvar, wcm, wcr = tn.group_timestep_norm_closed_form_full(x, pc, pm, pv, gamma, beta, m, H, 1e-5)
    assert torch.equal(count.cpu(), wcount) and cm.dtype == x.dtype and cm.shape == (B, L, H)
    assert rel_err(y, wy) <= 1e-4 and rel_err(mean, wmean) <= 1e-4 and rel_err(var, wvar) <= 1e-4
    assert rel_err(cm, wcm) <= 1e-4 and rel_err(cr, wcr) <= 1e-4
    got = ops.timestep_norm_bwd(*_cuda(dy, dmean, dvar, x, pm), count, cm, cr, gamma.cuda(),
                                None if m is None else m.cuda())
    want = tn.group_timestep_norm_bwd_autograd(dy, dmean, dvar, x, pc, pm, pv, gamma, beta, m, H, 1e-5)
    for name, a, b_ in zip(["dx", "dprev_mean", "dprev_var", "dgamma", "dbeta"], got, want):
        assert rel_err(a, b_) <= 1e-4, name


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mask", ["trailing", "holes"])
def test_padding_rows_are_never_read(mask, dtype):
    """NaN / Inf in x and dy at masked steps: every output agrees with a run with
    zeros there (masked steps have y = dx = 0, leave the statistics alone and
    add nothing to the parameter gradients).  Not bit for bit: the order in
    which a tile combines its predecessors' records varies from run to run."""
    B, L, H, G = 3, 333, 256, 4
    x, pc, pm, pv, gamma, beta, m, dy, dmean, dvar = _case(B, L, H, G, 21, dtype, 2, mask)
    clean_x, clean_dy = x.masked_fill(m.unsqueeze(-1), 0.0), dy.masked_fill(m.unsqueeze(-1), 0.0)
    junk = torch.where(torch.arange(H) % 2 == 0, float("nan"), float("inf")).to(dtype)
    dirty_x = torch.where(m.unsqueeze(-1), junk, x)
    dirty_dy = torch.where(m.unsqueeze(-1), -junk, dy)
    outs = []
    for xx, gg in ((clean_x, clean_dy), (dirty_x, dirty_dy)):
        cx, cpc, cpm, cpv, cg, cb, cm = _cuda(xx, pc, pm, pv, gamma, beta, m)
        fwd = ops.group_timestep_norm_fwd(cx, cpc, cpm, cpv, cg, cb, cm, G, 1e-5)
        y, count, mean, var, cummean, cumrstd = fwd
        bwd = ops.group_timestep_norm_bwd(gg.cuda(), dmean.cuda(), dvar.cuda(), cx, cpm, count, cummean, cumrstd,
                                          cg, cm, G)
        outs.append([t.cpu() for t in (*fwd, *bwd)])
    for a, b_ in zip(*outs):
        assert torch.isfinite(b_.float()).all()
        if a.dtype == torch.int64:
            assert torch.equal(a, b_)
        else:
            assert rel_err(b_, a.double()) <= (1e-5 if dtype == torch.float32 else 1e-2)
    assert (outs[1][0][m] == 0).all() and (outs[1][6][m] == 0).all()   # y and dx at masked steps


# A tile's wait for its predecessors' records is bounded.  The host forces the
# condition (one tile index publishes nothing, the poll limit is tiny): every
# kernel still exits, the status call reports the timeout, the outputs that
# depended on the missing record are NaN, and the next ordinary launch on the
# same workspace is clean again.
@pytest.mark.parametrize("H,G", [(256, 2), (1024, 2)])      # per-wave tiles / one workgroup per tile
def test_lookback_wait_is_bounded(H, G):
    from megalodon_amd import _lib
    B, L = 2, 64 * 6
    x, pc, pm, pv, gamma, beta, _, dy, dmean, dvar = _case(B, L, H, G, 3, torch.bfloat16, mask=None)
    args = _cuda(x, pc, pm, pv, gamma, beta)
    good = ops.group_timestep_norm_fwd(*args, None, G, 1e-5)
    ops.timestep_norm_status()
    hook = _lib.load().mega_test_timestep_norm_lookback
    hook.restype = None
    try:
        hook(_lib.ctypes.c_longlong(500), _lib.ctypes.c_int(2))
        y = ops.group_timestep_norm_fwd(*args, None, G, 1e-5)[0]
        with pytest.raises(RuntimeError, match="gave up waiting"):
            ops.timestep_norm_status()
        assert torch.equal(y[:, :64 * 3], good[0][:, :64 * 3])        # tiles 0..2 never needed tile 2's record
        assert torch.isnan(y[:, 64 * 3:].float()).all()               # tiles 3.. did
        dxm = ops.group_timestep_norm_bwd(*_cuda(dy, dmean, dvar, x, pm), good[1], good[4], good[5],
                                          args[4], None, G)[0]
        with pytest.raises(RuntimeError, match="gave up waiting"):
            ops.timestep_norm_status()
        assert torch.isnan(dxm[:, :64 * 2].float()).all()             # the backward runs from the end
    finally:
        hook(_lib.ctypes.c_longlong(0), _lib.ctypes.c_int(-1))
    again = ops.group_timestep_norm_fwd(*args, None, G, 1e-5)
    dx = ops.group_timestep_norm_bwd(*_cuda(dy, dmean, dvar, x, pm), again[1], again[4], again[5], args[4], None, G)[0]
    ops.timestep_norm_status()
    assert torch.equal(again[0], good[0]) and torch.isfinite(dx.float()).all()
