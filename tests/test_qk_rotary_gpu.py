"""The fused z -> (q, k) kernel (per-head RMSNorm, the two affine maps, rotary)
against float64 with autograd, rel err <= 2e-2 (bfloat16 / float16) for q, k and
the gradients of z, gamma, beta; then the block with rotary factors against the
float64 block oracle, and piecewise (cached) against the full pass."""
import math

import pytest
import torch

from conftest import rel_err
from megalodon_amd import extension as ops
from megalodon_amd.fused_ops import qk_norm_rotary
from megalodon_amd.modules import MegaBlock, RotaryEmbedding, apply_rotary_emb
from oracle import block as oblock

pytestmark = pytest.mark.gpu
TOL = 2e-2


def _oracle(z, gamma, beta, freqs, Dh, eps):
    B, L, S = z.shape
    H = S // Dh
    zz = z.view(B, L, H, Dh)
    zn = (zz * torch.rsqrt(zz.pow(2).mean(-1, keepdim=True) + eps)).view(B, L, S)
    u = zn.unsqueeze(2) * ((gamma + 1.0) / math.sqrt(Dh)) + beta
    q, k = torch.unbind(u, dim=2)
    if freqs is not None:
        P = freqs.shape[0]
        pos = torch.arange(L) % P
        f = freqs.to(torch.complex128)[pos]                      # L x Dh/2
        rot = lambda t: torch.view_as_real(torch.view_as_complex(t.reshape(B, L, H, Dh // 2, 2)) * f[None, :, None, :]).reshape(B, L, S)
        q, k = rot(q), rot(k)
    return q, k


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,L,S,Dh,P", [
    (2, 96, 1024, 256, 32),    # config-4 head layout; three chunks of 32 positions
    (1, 40, 512, 64, 40),      # a piece shorter than the chunk: one position per row
    (2, 33, 2048, 512, 0),     # no rotary
    (1, 50, 4096, 128, 25),
    (3, 7, 512, 512, 7),       # one head spanning the whole wavefront
])
def test_qk_norm_rotary_matches_float64(B, L, S, Dh, P, dtype):
    g = torch.Generator().manual_seed(S + Dh + L)
    z = (torch.randn(B, L, S, generator=g) * 2).to(dtype)
    gamma = (torch.randn(2, S, generator=g) * 0.3).to(dtype)
    beta = (torch.randn(2, S, generator=g) * 0.3).to(dtype)
    dq = torch.randn(B, L, S, generator=g).to(dtype)
    dk = torch.randn(B, L, S, generator=g).to(dtype)
    freqs = RotaryEmbedding(Dh, P).get_freqs_cis(0, P) if P else None
    zg, gg, bg = (t.cuda().requires_grad_(True) for t in (z, gamma, beta))
    q, k = qk_norm_rotary(zg, gg, bg, None if freqs is None else freqs.cuda(), Dh, 1e-5)
    (q.float() * dq.cuda().float() + k.float() * dk.cuda().float()).sum().backward()
    z64, g64, b64 = (t.double().requires_grad_(True) for t in (z, gamma, beta))
    wq, wk = _oracle(z64, g64, b64, freqs, Dh, 1e-5)
    (wq * dq.double() + wk * dk.double()).sum().backward()
    assert q.dtype == dtype and q.is_contiguous() and k.is_contiguous()
    assert rel_err(q, wq) <= TOL and rel_err(k, wk) <= TOL
    assert rel_err(zg.grad, z64.grad) <= TOL
    assert rel_err(gg.grad, g64.grad) <= TOL and rel_err(bg.grad, b64.grad) <= TOL


def test_rotary_part_equals_the_module_level_product():
    # with gamma = sqrt(Dh) - 1 and beta = 0 the kernel is znorm followed by the rotary product
    B, L, S, Dh, C = 2, 64, 512, 128, 16
    z = torch.randn(B, L, S, device="cuda").bfloat16()
    gamma = torch.full((2, S), math.sqrt(Dh) - 1.0, device="cuda").bfloat16()
    beta = torch.zeros(2, S, device="cuda").bfloat16()
    freqs = RotaryEmbedding(Dh, C).get_freqs_cis(0, C).cuda()
    q, k = ops.qk_norm_rotary_fwd(z, gamma, beta, freqs, Dh, 1e-5)[:2]
    zz = z.float().view(B, L, S // Dh, Dh)
    zn = (zz * torch.rsqrt(zz.pow(2).mean(-1, keepdim=True) + 1e-5)) * ((gamma[0, 0].float() + 1) / math.sqrt(Dh))
    want, _ = apply_rotary_emb(zn.view(B * L // C, C, S // Dh, Dh), zn.view(B * L // C, C, S // Dh, Dh), freqs)
    assert rel_err(q, want.reshape(B, L, S)) <= TOL and torch.equal(q, k)
    with pytest.raises(RuntimeError, match="head size"):
        ops.qk_norm_rotary_fwd(z[..., :384].contiguous(), gamma[:, :384].contiguous(), beta[:, :384].contiguous(),
                               None, 96, 1e-5)


def _block(chunk, heads=2):
    torch.manual_seed(3)
    blk = MegaBlock(model_dim=256, z_dim=512, value_dim=512, num_heads=heads, cema_ndim=16, chunk_size=chunk,
                    ffn_hidden_dim=384, norm_num_groups=4, init_std=0.05).cuda().bfloat16()
    with torch.no_grad():
        for n_, p_ in blk.named_parameters():
            if n_.endswith(("timenorm.weight", "timenorm.bias", "rmsnorm.weight", "mega.gamma", "mega.beta",
                            "norm.weight", "norm.bias", "wz.bias", "wv.bias", "wr.bias", "wh1.bias")):
                p_.normal_(0, 0.1)
    return blk


@pytest.mark.parametrize("rope", [False, True])
def test_block_on_the_fused_path_matches_the_float64_block(rope):
    chunk, B, L = 256, 2, 512
    blk = _block(chunk)
    freqs = RotaryEmbedding(256, chunk).get_freqs_cis(0, chunk) if rope else None
    g = torch.Generator().manual_seed(1)
    x = (torch.rand(B, L, 256, generator=g) * 2 - 1).bfloat16()
    dy = torch.randn(B, L, 256, generator=g).bfloat16()
    assert ops.qk_norm_rotary_supported(torch.empty(B, L, 512, device="cuda", dtype=torch.bfloat16), blk.mega.gamma, 256)
    xc = x.cuda().requires_grad_(True)
    out, _ = blk(xc, None if freqs is None else freqs.cuda())
    out.backward(dy.cuda())
    p = {n_: p_.detach().cpu().double().requires_grad_(True) for n_, p_ in blk.named_parameters()}
    xo = x.double().requires_grad_(True)
    want = oblock.mega_block_forward(p, xo, num_heads=2, ndim=16, chunk_size=chunk, groups=4, freqs_cis=freqs)
    want.backward(dy.double())
    assert rel_err(out, want) <= 5e-2 and rel_err(xc.grad, xo.grad) <= 5e-2
    for name in ("mega.gamma", "mega.beta", "mega.wz.weight", "mega.wv.weight", "mega.rmsnorm.weight",
                 "nffn.norm.weight", "nffn.norm.bias", "nffn.fc3.weight"):
        assert rel_err(dict(blk.named_parameters())[name].grad, p[name].grad) <= 5e-2, name
    if rope:   # the factors matter: without them the result moves
        out0, _ = blk(x.cuda())
        assert rel_err(out0, want) > 1e-3


def test_piecewise_with_rotary_equals_the_full_pass():
    chunk, bs = 256, 2
    blk = _block(chunk).eval()
    rope = RotaryEmbedding(256, chunk).cuda()
    x = torch.randn(bs, 2 * chunk, 256, device="cuda").bfloat16()
    m = blk.mega
    with torch.no_grad():
        full, _ = blk(x, rope.get_freqs_cis(0, chunk))
        k0 = torch.empty(bs, 0, m.local_heads, m.z_head_dim, dtype=torch.bfloat16, device="cuda")
        v0 = torch.empty(bs, 0, m.local_heads, m.v_head_dim, dtype=torch.bfloat16, device="cuda")
        cache = ((k0, v0, 0), (None, None, None), None)
        outs, pos = [], 0
        for n in [100, 156, 1, 1, 254]:
            start = pos % chunk
            y, cache = blk(x[:, pos:pos + n].contiguous(), rope.get_freqs_cis(start, min(start + n, chunk)), None, cache)
            outs.append(y)
            pos += n
    assert rel_err(torch.cat(outs, dim=1), full) <= TOL
