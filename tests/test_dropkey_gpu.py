"""DropKey attention dropout and the mask-free dropout operator on the GPU.

The masks are pure functions of (seed, offset, position) (include/megalodon_hip.h),
restated in oracle/philox.py and pinned there by Random123's known answers, so
the comparisons below are against the float64 oracle run with the same mask:
rel err <= 2e-2 for bfloat16 / float16 values and gradients, exact zeros where
a key was dropped, bit-exact results for the plain dropout operator.  The
reference draws its masks from curand's per-thread streams
(megalodon/csrc/softmax.cuh:161-171), which cannot be reproduced without its
thread layout: equality with the reference's own masks is not claimed."""
import numpy as np
import pytest
import torch

from conftest import rel_err
from megalodon_amd import extension as ops
from megalodon_amd.fused_ops import attention_softmax, memory_efficient_dropout, swift_efficient_attention
from megalodon_amd.fused_ops.memory_efficient_dropout import (memory_efficient_dropout_bwd,
                                                             memory_efficient_dropout_fwd)
from oracle import attention as oa
from oracle import philox

pytestmark = pytest.mark.gpu
TOL = 2e-2


def _generator_state():
    torch.cuda.init()
    gen = torch.cuda.default_generators[torch.cuda.current_device()]
    return gen.initial_seed(), gen.get_offset()


def _mask(B, NH, L1, L2, p, seed, offset):
    m = philox.dropkey_mask(np.arange(B * NH * L1), L2, p, seed, offset)
    return torch.from_numpy(m).view(B, NH, L1, L2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("B,L1,L2,NH,H1,H2,causal,p", [
    (2, 256, 256, 2, 64, 128, True, 0.1),      # one tile, rows in registers
    (1, 520, 1000, 2, 32, 64, True, 0.5),      # key/value prefix, three row tiles
    (2, 100, 131, 3, 32, 72, True, 0.3),       # ragged: the element-by-element softmax kernel
    (1, 300, 300, 1, 16, 24, False, 0.2),      # every row sees every key
    (1, 64, 4608, 1, 32, 32, False, 0.25),     # rows longer than the register-resident limit
])
def test_attention_with_dropkey_matches_the_oracle_under_the_same_mask(B, L1, L2, NH, H1, H2, causal, p, dtype):
    g = torch.Generator().manual_seed(L1 + L2)
    q = (torch.randn(B, L1, NH, H1, generator=g) / H1 ** 0.5).to(dtype)
    k = (torch.randn(B, L2, NH, H1, generator=g) / H1 ** 0.5).to(dtype)
    v = (torch.randn(B, L2, NH, H2, generator=g) / H2 ** 0.5).to(dtype)
    dy = torch.randn(B, L1, NH, H2, generator=g).to(dtype)
    TOL = 1e-4 if dtype == torch.float32 else globals()["TOL"]
    torch.manual_seed(77 + L1)
    seed, offset = _generator_state()
    y, w = ops.attention_fwd(q.cuda(), k.cuda(), v.cuda(), 0.7, p, causal)
    assert _generator_state()[1] > offset, "the launch must consume generator offsets"
    drop = _mask(B, NH, L1, L2, p, seed, offset)
    wy, wp = oa.chunk_attention_fwd(q, k, v, 0.7, causal, drop)
    wfull = torch.tril(w.float().cpu(), diagonal=L2 - L1) if causal else w.float().cpu()
    assert rel_err(y, wy) <= TOL and rel_err(wfull, wp) <= TOL
    # a dropped key has probability exactly 0, a kept one inside the causal range does not vanish
    visible = torch.ones(L1, L2, dtype=torch.bool).tril(diagonal=L2 - L1) if causal else torch.ones(L1, L2, dtype=torch.bool)
    assert (wfull[drop & visible] == 0).all()
    assert (wp[~drop & visible] > 0).all()
    dq, dk, dv = ops.attention_bwd(dy.cuda(), q.cuda(), k.cuda(), v.cuda(), w, 0.7, causal)
    wdq, wdk, wdv = oa.chunk_attention_bwd(dy, q, k, v, 0.7, causal, drop)
    assert rel_err(dq, wdq) <= TOL and rel_err(dk, wdk) <= TOL and rel_err(dv, wdv) <= TOL


def test_rows_that_lose_every_key_become_zero():
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(1, 96, 2, 32, generator=g).bfloat16().cuda() for _ in range(3))
    y, w = ops.attention_fwd(q, k, v, 1.0, 1.0, True)
    assert (w.float().tril() == 0).all() and (y == 0).all()
    dq, dk, dv = ops.attention_bwd(torch.ones_like(y), q, k, v, w, 1.0, True)
    assert (dq == 0).all() and (dk == 0).all() and (dv == 0).all()
    # at p = 0.6 row 0 (one key) is emptied in about 60 % of the matrices: zeros, never NaN
    q, k, v = (torch.randn(40, 8, 1, 16, generator=g).bfloat16().cuda() for _ in range(3))
    torch.manual_seed(11)
    seed, offset = _generator_state()
    y, w = ops.attention_fwd(q, k, v, 1.0, 0.6, True)
    drop = _mask(40, 1, 8, 8, 0.6, seed, offset)
    emptied = drop[:, 0, 0, 0]
    assert 10 < int(emptied.sum()) < 36
    assert torch.isfinite(y.float()).all() and torch.isfinite(w.float().tril()).all()
    assert (y[emptied.cuda(), 0] == 0).all() and (w[emptied.cuda(), 0, 0, 0] == 0).all()
    assert (w[~emptied.cuda(), 0, 0, 0] == 1).all()


def test_masks_follow_the_generator_and_drop_at_the_requested_rate():
    g = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(2, 512, 2, 32, generator=g).bfloat16().cuda() for _ in range(3))
    torch.manual_seed(123)
    _, w1 = ops.attention_fwd(q, k, v, 0.1, 0.2, False)
    _, w2 = ops.attention_fwd(q, k, v, 0.1, 0.2, False)
    torch.manual_seed(123)
    _, w3 = ops.attention_fwd(q, k, v, 0.1, 0.2, False)
    assert torch.equal(w1, w3) and not torch.equal(w1, w2)
    n = w1.numel()
    for w in (w1, w2):
        rate = float((w == 0).float().mean())
        assert abs(rate - 0.2) < 5 * (0.2 * 0.8 / n) ** 0.5
    # the autograd operator: dropout only while training
    torch.manual_seed(123)
    ya = swift_efficient_attention(q, k, v, 1.0, 0.2, False, True)
    yb = swift_efficient_attention(q, k, v, 1.0, 0.2, False, False)
    y0, _ = ops.attention_fwd(q, k, v, 1.0, 0.0, False)
    assert torch.equal(yb, y0) and not torch.equal(ya, y0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape,causal,p", [((3, 2, 64, 64), True, 0.3), ((2, 50, 77), True, 0.5),
                                            ((1, 16, 4104), False, 0.1), ((2, 24, 5000), True, 0.4)])
def test_standalone_softmax_with_dropkey(shape, causal, p, dtype):
    g = torch.Generator().manual_seed(shape[-1])
    x = (torch.randn(*shape, generator=g) * 2).to(dtype)
    dy = torch.randn(*shape, generator=g).to(dtype)
    L1, L2 = shape[-2], shape[-1]
    Z = x.numel() // (L1 * L2)
    torch.manual_seed(9)
    seed, offset = _generator_state()
    xg = x.cuda().requires_grad_(True)
    y = attention_softmax(xg, p, causal, True)
    y.backward(dy.cuda())
    drop = torch.from_numpy(philox.dropkey_mask(np.arange(Z * L1), L2, p, seed, offset)).view(shape)
    keep = ~drop
    if causal:
        r = torch.arange(L1).view(L1, 1)
        c = torch.arange(L2).view(1, L2)
        keep = keep & (c <= r + (L2 - L1))
    empty = ~keep.any(-1, keepdim=True)
    x64 = x.double().requires_grad_(True)
    want = torch.softmax(x64.masked_fill(~keep, float("-inf")).masked_fill(empty, 0.0), -1).masked_fill(empty, 0.0)
    want.backward(dy.double())
    assert rel_err(y, want) <= TOL
    assert (y.detach().cpu()[~keep] == 0).all()
    assert rel_err(xg.grad, x64.grad) <= TOL


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,p", [(8192, 0.1), (1003, 0.5), (5, 0.9), (3 * 4096 + 7, 0.25)])
def test_dropout_operator_is_bit_exact_and_needs_no_saved_mask(n, p, dtype):
    g = torch.Generator().manual_seed(n)
    x = torch.randn(n, generator=g).to(dtype)
    dy = torch.randn(n, generator=g).to(dtype)
    seed, offset = 0x0123456789ABCDEF, (3 << 32) + 40
    keep = torch.from_numpy(philox.dropout_keep(n, p, seed, offset))
    inv = torch.tensor(np.float32(1.0 / (1.0 - p)))
    want = torch.where(keep, (x.float() * inv).to(dtype), torch.zeros((), dtype=dtype))
    got = ops.dropout(x.cuda(), p, seed, offset)
    assert got.dtype == dtype and torch.equal(got.cpu(), want)
    # unaligned start: the element-by-element kernel draws the same mask
    xx = torch.cat([torch.zeros(1, dtype=dtype), x]).cuda()[1:]
    assert torch.equal(ops.dropout(xx, p, seed, offset).cpu(), want)
    # backward = the same call on the gradient
    y, state = memory_efficient_dropout_fwd(x.cuda(), p, True, rng_state=(seed, offset))
    assert state == (seed, offset) and torch.equal(y.cpu(), want)
    dx = memory_efficient_dropout_bwd(dy.cuda(), p, state)
    assert torch.equal(dx.cpu(), torch.where(keep, (dy.float() * inv).to(dtype), torch.zeros((), dtype=dtype)))


def test_memory_efficient_dropout_through_autograd():
    torch.manual_seed(31)
    x = torch.randn(4, 300, 64, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    y = memory_efficient_dropout(x, 0.3, True)
    kept = y != 0
    rate = 1.0 - float(kept.float().mean())
    assert abs(rate - 0.3) < 5 * (0.21 / x.numel()) ** 0.5 + 1e-3
    y.backward(torch.ones_like(y))
    assert torch.equal(x.grad != 0, kept)
    assert torch.equal(x.grad[kept], torch.full_like(x.grad[kept], 1 / 0.7))
    # identity when not training or p = 0, zeros at p = 1, errors outside [0, 1]
    assert memory_efficient_dropout(x, 0.3, False) is x and memory_efficient_dropout(x, 0.0, True) is x
    assert (memory_efficient_dropout(x, 1.0, True) == 0).all()
    with pytest.raises(ValueError):
        memory_efficient_dropout(x, 1.5, True)
    y2 = memory_efficient_dropout(x, 0.3, True)
    assert not torch.equal(y2 != 0, kept), "a second call must draw a new mask"


def test_block_with_all_three_dropouts():
    from megalodon_amd.modules import MegaBlock
    cfg = dict(model_dim=256, z_dim=64, value_dim=512, num_heads=2, cema_ndim=16, chunk_size=256,
               ffn_hidden_dim=384, norm_num_groups=4, init_std=0.05)
    torch.manual_seed(0)
    plain = MegaBlock(**cfg).cuda().bfloat16()
    noisy = MegaBlock(**cfg, dropout=0.1, attention_dropout=0.2, hidden_dropout=0.1).cuda().bfloat16()
    noisy.load_state_dict(plain.state_dict())
    x = (torch.rand(2, 512, 256, device="cuda") * 2 - 1).bfloat16()

    def run(block, seed):
        torch.manual_seed(seed)
        xi = x.clone().requires_grad_(True)
        block.zero_grad(set_to_none=True)
        out, _ = block(xi)
        out.float().pow(2).sum().backward()
        return out.detach(), xi.grad, block.mega.wv.weight.grad.clone()

    base = run(plain, 1)
    a, b, c = run(noisy, 1), run(noisy, 1), run(noisy, 2)
    for t in a:
        assert torch.isfinite(t.float()).all()
    assert all(torch.equal(u, v) for u, v in zip(a, b)), "same generator state, same masks"
    assert not torch.equal(a[0], c[0]) and not torch.equal(a[0], base[0])
    # dropout perturbs, it does not change the scale of the result
    assert 0.5 < float(a[0].float().abs().mean() / base[0].float().abs().mean()) < 2.0
    noisy.eval()
    with torch.no_grad():
        assert torch.equal(noisy(x)[0], plain(x)[0])
