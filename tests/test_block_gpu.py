"""One Megalodon block (TimestepNorm -> CEMA -> gated chunk attention ->
normalised FFN) in bf16 against the float64 composition of the oracles.
A whole block chains ~15 bf16-rounded operators, so the bar here is rel err
<= 5e-2 on the output and the gradients (each operator alone is held to 2e-2
in its own test)."""
import pytest
import torch

from conftest import rel_err
from megalodon_amd.modules import MegaBlock
from oracle import block as oblock

pytestmark = pytest.mark.gpu


def test_block_forward_backward_bf16():
    torch.manual_seed(0)
    cfg = dict(model_dim=256, z_dim=64, value_dim=512, num_heads=2, cema_ndim=16, chunk_size=256,
               ffn_hidden_dim=384, norm_num_groups=4)
    B, L = 2, 512
    blk = MegaBlock(**cfg, init_std=0.05).cuda().bfloat16()
    with torch.no_grad():   # move the zero-initialised affine parameters off zero
        for n_, p_ in blk.named_parameters():
            if n_.endswith(("timenorm.weight", "timenorm.bias", "rmsnorm.weight", "mega.gamma", "mega.beta",
                            "norm.weight", "norm.bias", "wz.bias", "wv.bias", "wr.bias", "wh1.bias")):
                p_.normal_(0, 0.1)
    g = torch.Generator().manual_seed(1)
    x = (torch.rand(B, L, cfg["model_dim"], generator=g) * 2 - 1).bfloat16()
    dy = torch.randn(B, L, cfg["model_dim"], generator=g).bfloat16()
    xc = x.cuda().requires_grad_(True)
    out, cache = blk(xc)
    assert cache is None and out.dtype == torch.bfloat16 and out.shape == x.shape
    out.backward(dy.cuda())

    p = {n_: p_.detach().cpu().double().requires_grad_(True) for n_, p_ in blk.named_parameters()}
    xo = x.double().requires_grad_(True)
    want = oblock.mega_block_forward(p, xo, num_heads=cfg["num_heads"], ndim=cfg["cema_ndim"],
                                     chunk_size=cfg["chunk_size"], groups=cfg["norm_num_groups"])
    want.backward(dy.double())
    assert rel_err(out, want) <= 5e-2
    assert rel_err(xc.grad, xo.grad) <= 5e-2
    for name in ("mega.cema.alpha", "mega.cema.delta", "mega.cema.theta", "mega.cema.gamma", "mega.cema.omega",
                 "mega.timenorm.weight", "mega.timenorm.bias", "mega.wz.weight", "mega.wv.weight",
                 "mega.wh2.weight", "nffn.fc1.weight"):
        got = dict(blk.named_parameters())[name].grad
        assert rel_err(got, p[name].grad) <= 5e-2, name
