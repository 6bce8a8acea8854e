"""Seeded synthetic inputs of the benchmark configurations.

All tensors are drawn on the CPU with ``torch.Generator().manual_seed(seed)``
and then cast / moved, so CPU and GPU runs see identical bits.
"""
from __future__ import annotations

import math
from typing import Dict

import torch


def cema_params(D: int, ndim: int, seed: int) -> Dict[str, torch.Tensor]:
    """Post-activation CEMA coefficients.

    alpha, delta = sigmoid(N(0,1)) per (D, ndim); theta ~ U(0, 2*pi/ndim) per D
    (mode n has angle theta*n, n = 1..ndim); gamma circular complex normal with
    total variance 1/ndim; omega ~ N(0,1) per D.
    Returns p (D,N,1) f32, q (D,N,1) c64, gamma (D,N) c64, omega (D,1) f32.
    """
    g = torch.Generator().manual_seed(seed)
    alpha = torch.sigmoid(torch.randn(D, ndim, 1, generator=g))
    delta = torch.sigmoid(torch.randn(D, ndim, 1, generator=g))
    theta = torch.rand(D, 1, 1, generator=g) * (2.0 * math.pi / ndim)
    wave = torch.arange(1, ndim + 1, dtype=torch.float32).view(1, ndim, 1)
    q = torch.polar(1.0 - alpha * delta, theta * wave)
    gam = torch.complex(torch.randn(D, ndim, generator=g), torch.randn(D, ndim, generator=g))
    gam = gam * math.sqrt(1.0 / (2.0 * ndim))
    omega = torch.randn(D, 1, generator=g)
    return {"p": alpha.contiguous(), "q": q.contiguous(), "gamma": gam.contiguous(), "omega": omega}


def cema_inputs(B: int, D: int, L: int, seed: int, dtype=torch.float32) -> Dict[str, torch.Tensor]:
    """x ~ N(0,1) (B, D, L) and an upstream gradient dy ~ N(0,1), cast to dtype."""
    g = torch.Generator().manual_seed(seed + 7919)
    x = torch.randn(B, D, L, generator=g).to(dtype)
    dy = torch.randn(B, D, L, generator=g).to(dtype)
    return {"x": x, "dy": dy}


def timestep_norm_inputs(B: int, L: int, D: int, G: int, seed: int, dtype=torch.bfloat16):
    """x = N(0,1) + c_d with c_d ~ N(0, 0.5) per channel; trailing padding mask
    with lengths U{L/2..L}; gamma ~ N(1, 0.02), beta ~ N(0, 0.02); prior
    count 0, mean 0, var 1; dy ~ N(0,1)."""
    g = torch.Generator().manual_seed(seed)
    offs = torch.randn(D, generator=g) * 0.5
    x = (torch.randn(B, L, D, generator=g) + offs).to(dtype)
    lengths = torch.randint(L // 2, L + 1, (B,), generator=g)
    mask = torch.arange(L).unsqueeze(0) >= lengths.unsqueeze(1)
    gamma = (1.0 + 0.02 * torch.randn(D, generator=g)).to(dtype)
    beta = (0.02 * torch.randn(D, generator=g)).to(dtype)
    dy = torch.randn(B, L, D, generator=g).to(dtype)
    return {
        "x": x, "mask": mask, "gamma": gamma, "beta": beta, "dy": dy,
        "prev_count": torch.zeros(B, dtype=torch.int64),
        "prev_mean": torch.zeros(B, G, dtype=dtype),
        "prev_var": torch.ones(B, G, dtype=dtype),
        "dmean": torch.zeros(B, G, dtype=dtype),
        "dvar": torch.zeros(B, G, dtype=dtype),
    }


def attention_inputs(Bc: int, C: int, heads: int, h1: int, h2: int, seed: int, dtype=torch.bfloat16):
    """q, k ~ N(0,1)/sqrt(h1) (Bc, C, heads, h1); v ~ N(0,1)/sqrt(h2); dy ~ N(0,1)."""
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(Bc, C, heads, h1, generator=g) / math.sqrt(h1)).to(dtype)
    k = (torch.randn(Bc, C, heads, h1, generator=g) / math.sqrt(h1)).to(dtype)
    v = (torch.randn(Bc, C, heads, h2, generator=g) / math.sqrt(h2)).to(dtype)
    dy = torch.randn(Bc, C, heads, h2, generator=g).to(dtype)
    return {"q": q, "k": k, "v": v, "dy": dy}
