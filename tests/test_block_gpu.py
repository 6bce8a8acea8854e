"""One Megalodon block (TimestepNorm -> CEMA -> gated chunk attention ->
normalised FFN) in bf16 against the float64 composition of the oracles.

Bars, rel err (max|a-b| / max|b|): <= 2e-2, the bar of the single operators, on the
output, on dx and on the gradients of the CEMA parameters (alpha, delta, theta,
gamma, omega); <= 3e-2 on the gradients of the other parameters, which pass through
up to fifteen bf16-rounded operators (measured on an MI355X: 5e-3 on the output,
9e-3 on dx, 5e-3 .. 9e-3 on the CEMA parameters, at most 2.1e-2 elsewhere -- the
q/k scale `mega.gamma` -- in the small block; the errors are printed, run with -s)."""
import pytest
import torch

from conftest import rel_err
from megalodon_amd.modules import MegaBlock, RotaryEmbedding
from oracle import block as oblock

pytestmark = pytest.mark.gpu
BAR = 2e-2
BAR_CHAIN = 3e-2
AFFINE = ("timenorm.weight", "timenorm.bias", "rmsnorm.weight", "mega.gamma", "mega.beta", "norm.weight", "norm.bias",
          "wz.bias", "wv.bias", "wr.bias", "wh1.bias")


def _block(cfg, seed):
    torch.manual_seed(seed)
    blk = MegaBlock(**cfg, init_std=0.05).cuda().bfloat16()
    with torch.no_grad():   # move the zero-initialised affine parameters off zero
        for n_, p_ in blk.named_parameters():
            if n_.endswith(AFFINE):
                p_.normal_(0, 0.1)
    return blk


def _against_oracle(blk, cfg, B, L, seed, freqs_cis=None):
    g = torch.Generator().manual_seed(seed)
    x = (torch.rand(B, L, cfg["model_dim"], generator=g) * 2 - 1).bfloat16()
    dy = torch.randn(B, L, cfg["model_dim"], generator=g).bfloat16()
    xc = x.cuda().requires_grad_(True)
    out, cache = blk(xc, None if freqs_cis is None else freqs_cis.cuda())
    assert cache is None and out.dtype == torch.bfloat16 and out.shape == x.shape
    out.backward(dy.cuda())

    p = {n_: p_.detach().cpu().double().requires_grad_(True) for n_, p_ in blk.named_parameters()}
    xo = x.double().requires_grad_(True)
    want = oblock.mega_block_forward(p, xo, num_heads=cfg["num_heads"], ndim=cfg["cema_ndim"],
                                     chunk_size=cfg["chunk_size"], groups=cfg["norm_num_groups"],
                                     freqs_cis=None if freqs_cis is None else freqs_cis.cpu())
    want.backward(dy.double())
    errs = {"out": rel_err(out, want), "dx": rel_err(xc.grad, xo.grad)}
    for name, prm in blk.named_parameters():
        errs["d " + name] = rel_err(prm.grad, p[name].grad)
    print("block errors vs float64 oracle:", {k: f"{v:.2e}" for k, v in errs.items()})
    return errs, (out, want)


def _over_the_bar(errs):
    tight = lambda k: k in ("out", "dx") or ".cema." in k
    return {k: v for k, v in errs.items() if not v <= (BAR if tight(k) else BAR_CHAIN)}


def test_block_forward_backward_bf16():
    cfg = dict(model_dim=256, z_dim=64, value_dim=512, num_heads=2, cema_ndim=16, chunk_size=256,
               ffn_hidden_dim=384, norm_num_groups=4)
    errs, _ = _against_oracle(_block(cfg, 0), cfg, B=2, L=512, seed=1)
    bad = _over_the_bar(errs)
    assert not bad, bad


def test_block_across_chunk_boundaries_with_rotary():
    """Four chunks of 1024 at width 512 (every attention product on its matrix-core kernels: head
    widths 128 / 512, key tiles beyond the first 256), rotary angles by position inside the chunk;
    the comparison with the oracle covers every chunk and both sides of each boundary."""
    cfg = dict(model_dim=512, z_dim=256, value_dim=1024, num_heads=2, cema_ndim=16, chunk_size=1024,
               ffn_hidden_dim=768, norm_num_groups=8)
    L = 4096
    rope = RotaryEmbedding(cfg["z_dim"] // cfg["num_heads"], cfg["chunk_size"])
    freqs = rope.get_freqs_cis(0, cfg["chunk_size"])
    errs, (out, want) = _against_oracle(_block(cfg, 2), cfg, B=1, L=L, seed=3, freqs_cis=freqs)
    bad = _over_the_bar(errs)
    assert not bad, bad
    # chunk by chunk, so that a chunk with small outputs cannot hide behind a large one
    C = cfg["chunk_size"]
    for c in range(L // C):
        assert rel_err(out[:, c * C:(c + 1) * C], want[:, c * C:(c + 1) * C]) <= BAR, c
    # the two tokens either side of every boundary
    for c in range(1, L // C):
        assert rel_err(out[:, c * C - 1:c * C + 1], want[:, c * C - 1:c * C + 1]) <= BAR, c
