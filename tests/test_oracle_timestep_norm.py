"""Pins the TimestepNorm oracle: brute-force prefix statistics, the closed form
with autograd, finite differences, and the reference's own C++ CPU path
(oracle/_ref, compiled from /root/reference) where it is built."""
import pytest
import torch

from oracle import native, timestep_norm as tn


def _case(B, L, H, G, seed, prior=3, mask="trailing"):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, L, H, generator=g, dtype=torch.float64) + 0.5 * torch.randn(H, generator=g, dtype=torch.float64)
    prev_count = torch.full((B,), prior, dtype=torch.int64)
    prev_mean = 0.3 * torch.randn(B, G, generator=g, dtype=torch.float64)
    prev_var = 0.5 + torch.rand(B, G, generator=g, dtype=torch.float64)
    gamma = 1.0 + 0.1 * torch.randn(H, generator=g, dtype=torch.float64)
    beta = 0.1 * torch.randn(H, generator=g, dtype=torch.float64)
    if mask == "trailing":
        lens = torch.randint(max(1, L // 2), L + 1, (B,), generator=g)
        m = torch.arange(L).unsqueeze(0) >= lens.unsqueeze(1)
    elif mask == "holes":
        m = torch.rand(B, L, generator=g) < 0.3
    else:
        m = None
    dy = torch.randn(B, L, H, generator=g, dtype=torch.float64)
    dmean = torch.randn(B, G, generator=g, dtype=torch.float64)
    dvar = torch.randn(B, G, generator=g, dtype=torch.float64)
    return x, prev_count, prev_mean, prev_var, gamma, beta, m, dy, dmean, dvar


def test_fwd_bruteforce_prefix_statistics_without_prior():
    """prev_count = 0: statistics at step t are the plain mean / biased variance of the
    per-step group means and second moments over the unmasked prefix."""
    B, L, H, G = 2, 13, 12, 3
    x, _, pm, pv, gamma, beta, m, *_ = _case(B, L, H, G, 1, mask="holes")
    pc = torch.zeros(B, dtype=torch.int64)
    eps = 1e-5
    y, count, mean, var, cm, cr = tn.group_timestep_norm_fwd(x, pc, pm, pv, gamma, beta, m, G, eps)
    D = H // G
    for b in range(B):
        seen = []
        for t in range(L):
            if not m[b, t]:
                seen.append(t)
            for g_ in range(G):
                if not seen:
                    assert cm[b, t, g_] == pm[b, g_]
                    continue
                blk = x[b, seen][:, g_ * D:(g_ + 1) * D]
                mu = blk.mean(dim=1)
                s2 = (blk * blk).mean(dim=1)
                U = mu.mean()
                V = s2.mean() - U * U
                assert abs(cm[b, t, g_] - U) < 1e-12
                assert abs(cr[b, t, g_] - 1 / torch.sqrt(V + eps)) < 1e-9
                if not m[b, t]:
                    want = (x[b, t, g_ * D:(g_ + 1) * D] - U) / torch.sqrt(V + eps) * gamma[g_ * D:(g_ + 1) * D] + beta[g_ * D:(g_ + 1) * D]
                    assert torch.allclose(y[b, t, g_ * D:(g_ + 1) * D], want, atol=1e-10)
                else:
                    assert y[b, t].abs().max() == 0
        assert count[b] == len(seen)


@pytest.mark.parametrize("mask", ["trailing", "holes", None])
@pytest.mark.parametrize("H,G", [(12, 3), (8, 8), (6, 1)])
def test_fwd_recursion_equals_closed_form(mask, H, G):
    x, pc, pm, pv, gamma, beta, m, *_ = _case(2, 17, H, G, 2, prior=5, mask=mask)
    y, count, mean, var, _, _ = tn.group_timestep_norm_fwd(x, pc, pm, pv, gamma, beta, m, G, 1e-5)
    y2, mean2, var2 = tn.group_timestep_norm_closed_form(x, pc, pm, pv, gamma, beta, m, G, 1e-5)
    assert torch.allclose(y, y2, atol=1e-11)
    assert torch.allclose(mean, mean2, atol=1e-12) and torch.allclose(var, var2, atol=1e-12)
    nvalid = 17 if m is None else (~m).sum(1)
    assert torch.equal(count, pc + nvalid)


@pytest.mark.parametrize("mask", ["trailing", "holes", None])
@pytest.mark.parametrize("H,G", [(12, 3), (8, 8), (6, 1)])
def test_bwd_recurrence_equals_autograd(mask, H, G):
    x, pc, pm, pv, gamma, beta, m, dy, dmean, dvar = _case(2, 15, H, G, 3, prior=4, mask=mask)
    y, count, mean, var, cm, cr = tn.group_timestep_norm_fwd(x, pc, pm, pv, gamma, beta, m, G, 1e-5)
    got = tn.group_timestep_norm_bwd(dy, dmean, dvar, x, pm, count, cm, cr, gamma, m, G)
    want = tn.group_timestep_norm_bwd_autograd(dy, dmean, dvar, x, pc, pm, pv, gamma, beta, m, G, 1e-5)
    for a, b_ in zip(got, want):
        assert torch.allclose(a, b_, atol=1e-10)


def test_bwd_finite_differences():
    B, L, H, G = 1, 6, 4, 2
    x, pc, pm, pv, gamma, beta, m, dy, dmean, dvar = _case(B, L, H, G, 4, prior=2, mask="trailing")
    y, count, mean, var, cm, cr = tn.group_timestep_norm_fwd(x, pc, pm, pv, gamma, beta, m, G, 1e-5)
    dx, dpm, dpv, dg, db = tn.group_timestep_norm_bwd(dy, dmean, dvar, x, pm, count, cm, cr, gamma, m, G)

    def loss(x_, pm_, pv_):
        y_, _, mean_, var_, _, _ = tn.group_timestep_norm_fwd(x_, pc, pm_, pv_, gamma, beta, m, G, 1e-5)
        return ((y_ * dy).sum() + (mean_ * dmean).sum() + (var_ * dvar).sum()).item()

    h = 1e-6
    for idx in [(0, 0, 0), (0, 2, 3), (0, 1, 1)]:
        e = torch.zeros_like(x)
        e[idx] = h
        fd = (loss(x + e, pm, pv) - loss(x - e, pm, pv)) / (2 * h)
        assert abs(fd - dx[idx].item()) < 1e-6
    e = torch.zeros_like(pm)
    e[0, 1] = h
    assert abs((loss(x, pm + e, pv) - loss(x, pm - e, pv)) / (2 * h) - dpm[0, 1].item()) < 1e-6
    assert abs((loss(x, pm, pv + e) - loss(x, pm, pv - e)) / (2 * h) - dpv[0, 1].item()) < 1e-6


def _check_native(lib, prefix, mask):
    B, L, H, G = 3, 40, 24, 4
    x, pc, pm, pv, gamma, beta, m, dy, dmean, dvar = _case(B, L, H, G, 7, prior=6, mask=mask)
    f = lambda t: t.float()
    got = native.group_timestep_norm_fwd(lib, prefix, f(x), pc, f(pm), f(pv), f(gamma), f(beta), m, G, 1e-5)
    want = tn.group_timestep_norm_fwd(f(x), pc, f(pm), f(pv), f(gamma), f(beta), m, G, 1e-5)
    names = ["y", "count", "mean", "var", "cummean", "cumrstd"]
    valid = torch.ones(B, L, 1, dtype=torch.bool) if m is None else (~m).unsqueeze(-1)
    for n_, a, b_ in zip(names, got, want):
        if n_ == "count":
            assert torch.equal(a, b_)
        elif n_ in ("cummean", "cumrstd") and prefix == "ref_":
            # the reference CPU loop stores the would-be-updated statistics at
            # masked steps (timestep_norm.cc:294-297): compare unmasked steps only
            assert ((a.double() - b_) * valid).abs().max() / b_.abs().max() < 2e-5, n_
        else:
            assert (a.double() - b_).abs().max() / b_.abs().max() < 2e-5, n_
    y, count, mean, var, cm, cr = want
    # each implementation consumes its own saved statistics
    gb = native.group_timestep_norm_bwd(lib, prefix, f(dy), f(dmean), f(dvar), f(x), f(pm), got[1], got[4], got[5], f(gamma), m, G)
    wb = tn.group_timestep_norm_bwd(f(dy), f(dmean), f(dvar), f(x), f(pm), count, cm, cr, f(gamma), m, G)
    for n_, a, b_ in zip(["dx", "dprev_mean", "dprev_var", "dgamma", "dbeta"], gb, wb):
        assert (a.double() - b_).abs().max() / b_.abs().max() < 1e-4, n_


@pytest.mark.parametrize("mask", ["trailing", "holes", None])
def test_c_port_matches_oracle(mask):
    _check_native(native.port(), "oracle_", mask)


@pytest.mark.skipif(native.ref() is None, reason="oracle/_ref not built (needs /root/reference)")
@pytest.mark.parametrize("mask", ["trailing", None])
def test_reference_cpp_cpu_path_matches_oracle(mask):
    """GroupTimestepNormCPUFwd/Bwd compiled from the reference's own sources.
    Trailing padding / no mask only: at interior masked steps the reference's
    CPU loop and its CUDA kernel store different cummean (see oracle header)."""
    _check_native(native.ref(), "ref_", mask)
