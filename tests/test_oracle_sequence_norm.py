"""Pins the sequence-norm oracle: torch's group_norm (the unmasked operator is
exactly group normalisation of the (B, H, L) tensor), a brute-force evaluation
on the unmasked steps alone, autograd, and the reference's own C++ CPU path
(oracle/_ref, compiled from /root/reference) where it is built."""
import pytest
import torch
import torch.nn.functional as F

from oracle import native, sequence_norm as sn


def _case(B, L, H, seed, mask="holes", length_last=False):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, L, H, generator=g, dtype=torch.float64) * 1.5 + torch.randn(H, generator=g, dtype=torch.float64)
    dy = torch.randn(B, L, H, generator=g, dtype=torch.float64)
    gamma = 1.0 + 0.3 * torch.randn(H, generator=g, dtype=torch.float64)
    beta = 0.2 * torch.randn(H, generator=g, dtype=torch.float64)
    if mask == "holes":
        m = torch.rand(B, L, generator=g) < 0.3
        m[:, 0] = False
    elif mask == "trailing":
        lens = torch.randint(1, L + 1, (B,), generator=g)
        m = torch.arange(L).unsqueeze(0) >= lens.unsqueeze(1)
    else:
        m = None
    if length_last:
        x, dy = x.transpose(1, 2).contiguous(), dy.transpose(1, 2).contiguous()
    return x, dy, gamma, beta, m


@pytest.mark.parametrize("G", [1, 3, 12])
@pytest.mark.parametrize("length_last", [False, True])
def test_unmasked_forward_is_group_norm(G, length_last):
    B, L, H = 3, 37, 12
    x, _, gamma, beta, _ = _case(B, L, H, 1, mask=None, length_last=length_last)
    y, count, mean, rstd = sn.group_sequence_norm_fwd(x, gamma, beta, None, G, 1e-5, length_last)
    xc = x if length_last else x.transpose(1, 2)
    want = F.group_norm(xc, G, gamma, beta, 1e-5)
    want = want if length_last else want.transpose(1, 2)
    assert torch.allclose(y, want, atol=1e-12)
    assert (count == L).all()
    grp = xc.reshape(B, G, -1)
    assert torch.allclose(mean, grp.mean(2), atol=1e-12)
    assert torch.allclose(rstd, 1 / torch.sqrt(grp.var(2, unbiased=False) + 1e-5), atol=1e-12)


@pytest.mark.parametrize("mask", ["holes", "trailing"])
@pytest.mark.parametrize("length_last", [False, True])
def test_masked_forward_equals_group_norm_of_the_kept_steps(mask, length_last):
    B, L, H, G = 3, 29, 8, 2
    x, _, gamma, beta, m = _case(B, L, H, 2, mask=mask, length_last=length_last)
    y, count, mean, rstd = sn.group_sequence_norm_fwd(x, gamma, beta, m, G, 1e-5, length_last)
    xb = x.transpose(1, 2) if length_last else x
    yb = y.transpose(1, 2) if length_last else y
    for b in range(B):
        keep = ~m[b]
        assert count[b] == keep.sum()
        kept = xb[b, keep]  # (n, H)
        want = F.group_norm(kept.t().unsqueeze(0), G, gamma, beta, 1e-5)[0].t()
        assert torch.allclose(yb[b, keep], want, atol=1e-12)
        assert yb[b, ~keep].abs().max() == 0 if (~keep).any() else True


@pytest.mark.parametrize("G", [1, 2, 8])
@pytest.mark.parametrize("length_last", [False, True])
def test_backward_matches_autograd(G, length_last):
    B, L, H = 2, 23, 8
    x, dy, gamma, beta, m = _case(B, L, H, 3, length_last=length_last)
    xr, gr, br = x.clone().requires_grad_(), gamma.clone().requires_grad_(), beta.clone().requires_grad_()
    y, count, mean, rstd = sn.group_sequence_norm_fwd(xr, gr, br, m, G, 1e-5, length_last)
    y.backward(dy)
    dx, dg, db = sn.group_sequence_norm_bwd(dy, x, count, mean.detach(), rstd.detach(), gamma, m, G, length_last)
    assert torch.allclose(dx, xr.grad, atol=1e-11)
    assert torch.allclose(dg, gr.grad, atol=1e-11)
    assert torch.allclose(db, br.grad, atol=1e-11)


def test_fully_masked_sequence():
    B, L, H, G = 2, 9, 6, 3
    x, dy, gamma, beta, m = _case(B, L, H, 4)
    m[1] = True
    y, count, mean, rstd = sn.group_sequence_norm_fwd(x, gamma, beta, m, G, 1e-5)
    assert count[1] == 0 and y[1].abs().max() == 0 and mean[1].abs().max() == 0
    dx, dg, db = sn.group_sequence_norm_bwd(dy, x, count, mean, rstd, gamma, m, G)
    assert dx[1].abs().max() == 0 and torch.isfinite(dg).all()


@pytest.mark.parametrize("G", [2, 8])
@pytest.mark.parametrize("length_last", [False, True])
@pytest.mark.parametrize("mask", ["holes", None])
def test_against_reference_cpu_build(G, length_last, mask):
    lib = native.ref()
    if lib is None or not hasattr(lib, "ref_group_sequence_norm_fwd"):
        pytest.skip("oracle/_ref is not built with sequence_norm.cc")
    B, L, H = 3, 300, 8
    x, dy, gamma, beta, m = _case(B, L, H, 5, mask=mask, length_last=length_last)
    y, count, mean, rstd = sn.group_sequence_norm_fwd(x, gamma, beta, m, G, 1e-5, length_last)
    ry, rcount, rmean, rrstd = native.group_sequence_norm_fwd(lib, x, gamma, beta, m, G, 1e-5, length_last)
    assert torch.equal(count, rcount)
    assert torch.allclose(y.float(), ry, atol=2e-5, rtol=1e-5)
    assert torch.allclose(mean.float(), rmean, atol=1e-5)
    assert torch.allclose(rstd.float(), rrstd, rtol=1e-5)
    dx, dg, db = sn.group_sequence_norm_bwd(dy, x, count, mean, rstd, gamma, m, G, length_last)
    rdx, rdg, rdb = native.group_sequence_norm_bwd(lib, dy, x, rcount, rmean, rrstd, gamma, m, G, length_last)
    assert torch.allclose(dx.float(), rdx, atol=5e-5, rtol=1e-4)
    assert torch.allclose(dg.float(), rdg, atol=2e-3, rtol=1e-4)
    assert torch.allclose(db.float(), rdb, atol=2e-4, rtol=1e-4)
