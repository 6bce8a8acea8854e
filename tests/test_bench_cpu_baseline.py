"""The float32 CPU baseline that bench.py times beside the GPU block (`cpu_block_forward`: the
reference's CPU formulation of every stage) computes the block: its output and gradients agree
with the float64 oracle of the block at a small shape (bar 1e-4, float32 arithmetic)."""
import os
import sys

import torch

from conftest import rel_err
from oracle import block as oblock

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import bench  # noqa: E402


def test_cpu_block_baseline_matches_block_oracle():
    cfg = dict(model_dim=64, z_dim=32, value_dim=128, num_heads=2, cema_ndim=16, chunk_size=256,
               ffn_hidden_dim=96, norm_num_groups=4)
    D, Z, H, F_, N, L = 64, 32, 128, 96, 16, 200
    g = torch.Generator().manual_seed(7)
    r = lambda *s: (torch.randn(*s, generator=g) * 0.3).requires_grad_(True)
    shapes = {"mega.timenorm.weight": (D,), "mega.timenorm.bias": (D,), "mega.cema.alpha": (D, N, 1),
              "mega.cema.delta": (D, N, 1), "mega.cema.theta": (D, 1, 1), "mega.cema.gamma": (D, N, 2),
              "mega.cema.omega": (D, 1), "mega.rmsnorm.weight": (D,), "mega.wz.weight": (Z, D), "mega.wz.bias": (Z,),
              "mega.wv.weight": (H, D), "mega.wv.bias": (H,), "mega.wr.weight": (H, D), "mega.wr.bias": (H,),
              "mega.wh1.weight": (D, D), "mega.wh1.bias": (D,), "mega.wh2.weight": (D, H), "mega.gamma": (2, Z),
              "mega.beta": (2, Z), "nffn.norm.weight": (D,), "nffn.norm.bias": (D,), "nffn.fc1.weight": (F_, D),
              "nffn.fc2.weight": (D, F_), "nffn.fc3.weight": (F_, D)}
    p = {k: r(*s) for k, s in shapes.items()}
    x = (torch.rand(1, L, D, generator=g) * 2 - 1).requires_grad_(True)
    dy = torch.randn(1, L, D, generator=g)
    out = bench.cpu_block_forward(p, x, cfg)
    out.backward(dy)

    p64 = {k: v.detach().double().requires_grad_(True) for k, v in p.items()}
    x64 = x.detach().double().requires_grad_(True)
    want = oblock.mega_block_forward(p64, x64, num_heads=2, ndim=N, chunk_size=256, groups=4)
    want.backward(dy.double())
    assert rel_err(out, want) <= 1e-4
    assert rel_err(x.grad, x64.grad) <= 1e-4
    for k in p:
        assert rel_err(p[k].grad, p64[k].grad) <= 1e-4, k
