"""Oracle for the group TimestepNorm (float64).

Follows megalodon/csrc/ops/timestep_norm.cc:218-316 (forward) and :318-450
(backward) with the merge operator of megalodon/csrc/utils.h:154-164, and the
module defaults of megalodon/modules/timestep_norm.py:106-126.

Masked steps: the state is left unchanged, y = 0, and the stored
cummean/cumrstd are those of the unchanged state -- the behaviour of the
reference's CUDA kernels (timestep_norm_kernel.cu:621-626).  The reference's
CPU loop stores the would-be-updated mean at masked steps instead
(timestep_norm.cc:294-297); both agree when the mask is trailing padding.
"""
from __future__ import annotations

import torch


def group_timestep_norm_fwd(x, prev_count, prev_mean, prev_var, gamma, beta, padding_mask, num_groups, eps):
    """Step-by-step restatement (loops over time).  Returns
    (y, count, mean, var, cummean, cumrstd), all float64 except count."""
    B, L, H = x.shape
    G = num_groups
    D = H // G
    x = x.double()
    gamma = gamma.double()
    beta = beta.double()
    xg = x.view(B, L, G, D)
    gu = xg.mean(dim=-1)
    gv = xg.var(dim=-1, unbiased=False)
    y = torch.zeros_like(x)
    cummean = torch.zeros(B, L, G, dtype=torch.float64)
    cumrstd = torch.zeros(B, L, G, dtype=torch.float64)
    count = prev_count.clone().to(torch.int64)
    mean = prev_mean.double().clone()
    var = prev_var.double().clone()
    for b in range(B):
        m0 = int(prev_count[b])
        u = prev_mean[b].double().clone()
        v = prev_var[b].double().clone()
        for j in range(L):
            masked = padding_mask is not None and bool(padding_mask[b, j])
            if not masked:
                # WelfordCombine(m0, u, v, 1, gu, gv)   utils.h:154-164
                n = m0 + 1
                c1 = m0 / n
                c2 = 1.0 / n
                delta = gu[b, j] - u
                u = c1 * u + c2 * gu[b, j]
                v = c1 * v + c2 * gv[b, j] + (c1 * delta) * (c2 * delta)
                m0 = n
            rstd = 1.0 / torch.sqrt(v + eps)
            cummean[b, j] = u
            cumrstd[b, j] = rstd
            if not masked:
                yy = (xg[b, j] - u.unsqueeze(-1)) * rstd.unsqueeze(-1)
                y[b, j] = yy.reshape(H) * gamma + beta
        count[b] = m0
        mean[b] = u
        var[b] = v
    return y, count, mean, var, cummean, cumrstd


def group_timestep_norm_closed_form(x, prev_count, prev_mean, prev_var, gamma, beta, padding_mask, num_groups, eps):
    """Vectorised closed form (differentiable):  with w_t = 1 - mask_t,
    n_t = n0 + sum_{tau<=t} w,  U_t = (n0 u0 + sum w mu)/n_t,
    Q_t = (n0 (v0 + u0^2) + sum w s)/n_t,  V_t = Q_t - U_t^2  (mu, s = group mean
    of x and x^2).  Returns (y, mean, var)."""
    B, L, H = x.shape
    G = num_groups
    D = H // G
    xg = x.view(B, L, G, D)
    mu = xg.mean(dim=-1)
    s2 = (xg * xg).mean(dim=-1)
    if padding_mask is None:
        w = torch.ones(B, L, dtype=x.dtype)
    else:
        w = (~padding_mask).to(x.dtype)
    n0 = prev_count.to(x.dtype).view(B, 1)
    n = n0 + torch.cumsum(w, dim=1)  # (B, L)
    nn = n.clamp(min=1.0).unsqueeze(-1)
    u0 = prev_mean.view(B, 1, G)
    v0 = prev_var.view(B, 1, G)
    U = (n0.unsqueeze(-1) * u0 + torch.cumsum(w.unsqueeze(-1) * mu, dim=1)) / nn
    Q = (n0.unsqueeze(-1) * (v0 + u0 * u0) + torch.cumsum(w.unsqueeze(-1) * s2, dim=1)) / nn
    V = Q - U * U
    # an all-masked prefix with n0 == 0 keeps the prior untouched
    empty = (n == 0).unsqueeze(-1)
    U = torch.where(empty, u0.expand_as(U), U)
    V = torch.where(empty, v0.expand_as(V), V)
    r = 1.0 / torch.sqrt(V + eps)
    y = ((xg - U.unsqueeze(-1)) * r.unsqueeze(-1)).reshape(B, L, H) * gamma + beta
    y = y * w.unsqueeze(-1)
    return y, U[:, -1], V[:, -1]


def group_timestep_norm_bwd(dy, dmean, dvar, x, prev_mean, count, cummean, cumrstd, gamma, padding_mask, num_groups):
    """Reverse-time recurrence restating timestep_norm.cc:385-430.  Returns
    (dx, dprev_mean, dprev_var, dgamma, dbeta) in float64."""
    B, L, H = x.shape
    G = num_groups
    D = H // G
    x = x.double().view(B, L, G, D)
    dy = dy.double().view(B, L, G, D)
    gam = gamma.double().view(G, D)
    cummean = cummean.double()
    cumrstd = cumrstd.double()
    dx = torch.zeros(B, L, G, D, dtype=torch.float64)
    dgamma = torch.zeros(G, D, dtype=torch.float64)
    dbeta = torch.zeros(G, D, dtype=torch.float64)
    dpm = torch.zeros(B, G, dtype=torch.float64)
    dpv = torch.zeros(B, G, dtype=torch.float64)
    cg = 1.0 / D
    for b in range(B):
        m0 = int(count[b])
        ug = dmean[b].double().clone()
        vg = dvar[b].double().clone()
        for j in range(L - 1, -1, -1):
            masked = padding_mask is not None and bool(padding_mask[b, j])
            if masked:
                continue
            c1 = (m0 - 1) / m0
            c2 = 1.0 / m0
            m0 -= 1
            prev_u = prev_mean[b].double() if j == 0 else cummean[b, j - 1]
            u = cummean[b, j]
            r = cumrstd[b, j]
            ux = x[b, j].mean(dim=-1)
            ds = (dy[b, j] * (x[b, j] - u.unsqueeze(-1)) * gam).sum(-1)
            db = (dy[b, j] * gam).sum(-1)
            du = ug - r * db
            dv = vg - 0.5 * r ** 3 * ds
            dux = c2 * du + 2.0 * c1 * c2 * dv * (ux - prev_u)
            dvx = c2 * dv
            dx[b, j] = (dy[b, j] * r.unsqueeze(-1) * gam + dux.unsqueeze(-1) * cg
                        + 2.0 * dvx.unsqueeze(-1) * cg * (x[b, j] - ux.unsqueeze(-1)))
            dgamma += dy[b, j] * (x[b, j] - u.unsqueeze(-1)) * r.unsqueeze(-1)
            dbeta += dy[b, j]
            ug = c1 * du - 2.0 * c1 * c2 * dv * (ux - prev_u)
            vg = c1 * dv
        dpm[b] = ug
        dpv[b] = vg
    return dx.view(B, L, H), dpm, dpv, dgamma.view(H), dbeta.view(H)


def group_timestep_norm_bwd_autograd(dy, dmean, dvar, x, prev_count, prev_mean, prev_var, gamma, beta,
                                     padding_mask, num_groups, eps):
    """Gradients by autograd over the closed form (fast for large L)."""
    x = x.double().requires_grad_(True)
    pm = prev_mean.double().requires_grad_(True)
    pv = prev_var.double().requires_grad_(True)
    g = gamma.double().requires_grad_(True)
    bt = beta.double().requires_grad_(True)
    y, mean, var = group_timestep_norm_closed_form(x, prev_count, pm, pv, g, bt, padding_mask, num_groups, eps)
    loss = (y * dy.double()).sum() + (mean * dmean.double()).sum() + (var * dvar.double()).sum()
    loss.backward()
    return x.grad, pm.grad, pv.grad, g.grad, bt.grad


def group_timestep_norm_closed_form_full(x, prev_count, prev_mean, prev_var, gamma, beta, padding_mask,
                                         num_groups, eps):
    """Closed form returning everything the operator returns, in float64:
    (y, count, mean, var, cummean, cumrstd).  Vectorised (fast at L = 8192)."""
    B, L, H = x.shape
    G = num_groups
    D = H // G
    x = x.double()
    xg = x.view(B, L, G, D)
    mu = xg.mean(dim=-1)
    s2 = (xg * xg).mean(dim=-1)
    w = torch.ones(B, L, dtype=torch.float64) if padding_mask is None else (~padding_mask).double()
    n0 = prev_count.double().view(B, 1)
    n = n0 + torch.cumsum(w, dim=1)
    nn = n.clamp(min=1.0).unsqueeze(-1)
    u0 = prev_mean.double().view(B, 1, G)
    v0 = prev_var.double().view(B, 1, G)
    U = (n0.unsqueeze(-1) * u0 + torch.cumsum(w.unsqueeze(-1) * mu, dim=1)) / nn
    Q = (n0.unsqueeze(-1) * (v0 + u0 * u0) + torch.cumsum(w.unsqueeze(-1) * s2, dim=1)) / nn
    V = Q - U * U
    empty = (n == 0).unsqueeze(-1)
    U = torch.where(empty, u0.expand_as(U), U)
    V = torch.where(empty, v0.expand_as(V), V)
    r = 1.0 / torch.sqrt(V + eps)
    y = ((xg - U.unsqueeze(-1)) * r.unsqueeze(-1)).reshape(B, L, H) * gamma.double() + beta.double()
    y = y * w.unsqueeze(-1)
    count = prev_count.to(torch.int64) + w.sum(dim=1).to(torch.int64)
    return y, count, U[:, -1], V[:, -1], U, r
