"""Parity of the HIP chunk attention with the float64 oracle.  Tolerance:
rel err (max|a-b|/max|b|) <= 2e-2 for bfloat16 / float16 tensors (forward
values and the gradients of q, k, v)."""
import pytest
import torch

from conftest import rel_err
from megalodon_amd import extension as ops
from megalodon_amd import synthetic
from megalodon_amd.fused_ops import swift_efficient_attention
from megalodon_amd.modules import _InnerAttention
from oracle import attention as oa

pytestmark = pytest.mark.gpu
TOL = 2e-2
TOL_F32 = 1e-4   # float32 tensors (the vector-ALU flavour of the operator)
TOL_F64 = 1e-12  # float64 tensors (the same flavour in double precision)


def _run(B, L1, L2, NH, H1, H2, causal, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, L1, NH, H1, generator=g) / H1 ** 0.5).to(dtype)
    k = (torch.randn(B, L2, NH, H1, generator=g) / H1 ** 0.5).to(dtype)
    v = (torch.randn(B, L2, NH, H2, generator=g) / H2 ** 0.5).to(dtype)
    dy = torch.randn(B, L1, NH, H2, generator=g).to(dtype)
    TOL = {torch.float32: TOL_F32, torch.float64: TOL_F64}.get(dtype, globals()["TOL"])
    y, w = ops.attention_fwd(q.cuda(), k.cuda(), v.cuda(), scale, 0.0, causal)
    wy, wp = oa.chunk_attention_fwd(q, k, v, scale, causal)
    assert y.shape == (B, L1, NH, H2) and w.shape == (B, NH, L1, L2) and y.dtype == dtype and w.dtype == dtype
    assert rel_err(y, wy) <= TOL
    # every row of w is written to its end, as the reference's softmax does
    # (softmax.cuh:99-105,127-129): exact zeros behind the causal limit
    assert rel_err(w, wp) <= TOL
    if causal:
        assert not torch.triu(w, diagonal=L2 - L1 + 1).any()
        # `lower_only`: what the backward reads is the same, the rest of w is undefined
        y2, w2 = ops.attention_fwd(q.cuda(), k.cuda(), v.cuda(), scale, 0.0, causal, lower_only=True)
        assert torch.equal(y2, y) and torch.equal(torch.tril(w2, diagonal=L2 - L1), torch.tril(w, diagonal=L2 - L1))
        got = ops.attention_bwd(dy.cuda(), q.cuda(), k.cuda(), v.cuda(), w2, scale, causal)
    dq, dk, dv = ops.attention_bwd(dy.cuda(), q.cuda(), k.cuda(), v.cuda(), w, scale, causal)
    wdq, wdk, wdv = oa.chunk_attention_bwd(dy, q, k, v, scale, causal)
    assert rel_err(dq, wdq) <= TOL and rel_err(dk, wdk) <= TOL and rel_err(dv, wdv) <= TOL
    if causal:
        assert all(torch.equal(a, b) for a, b in zip(got, (dq, dk, dv)))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,L,NH,H1,H2", [
    (2, 256, 2, 64, 128),     # exactly one tile
    (1, 512, 1, 256, 256),    # 2x2 tiles: off-diagonal tile skipping
    (2, 300, 3, 32, 72),      # ragged edges in every dimension
    (1, 1024, 2, 256, 512),   # config-3 head dims (qk 256), shorter chunk
    (3, 50, 2, 16, 24),       # tiny, rows not multiples of 8 (unaligned operand path)
    (1, 1, 1, 8, 8),          # single query
])
def test_causal_fwd_bwd(B, L, NH, H1, H2, dtype):
    _run(B, L, L, NH, H1, H2, True, dtype, seed=L + H2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,L1,L2,NH,H1,H2", [
    (2, 212, 512, 2, 64, 128),    # cached keys in front: diagonal shifted by 300 columns
    (1, 256, 768, 1, 256, 256),   # shift by two whole tiles
    (1, 520, 1000, 2, 32, 64),    # three row tiles, shift not a multiple of the k slab
    (2, 100, 131, 3, 32, 72),     # ragged, unaligned operand path
    (1, 1, 40, 1, 16, 16),        # one new query, causal flag kept: sees all keys
    (1, 1024, 1280, 1, 256, 512), # config-3 head dims, prefix of 256
])
def test_causal_with_key_value_prefix(B, L1, L2, NH, H1, H2, dtype):
    """L2 > L1: row r attends to keys 0 .. L2 - L1 + r (bottom-right aligned
    mask), forward values, probabilities and all three gradients."""
    _run(B, L1, L2, NH, H1, H2, True, dtype, seed=L1 + L2)


@pytest.mark.parametrize("B,L1,L2,NH,H1,H2,causal", [
    (2, 256, 256, 2, 64, 128, True),     # whole 64 x 64 tiles
    (2, 100, 131, 3, 32, 72, True),      # ragged in every dimension, key/value prefix
    (1, 300, 300, 1, 16, 24, False),     # every row sees every key
    (1, 1, 40, 1, 16, 16, True),         # one new query
    (1, 520, 1000, 2, 32, 64, True),     # several row tiles, prefix of 480 keys
])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_float32_and_float64_tensors(B, L1, L2, NH, H1, H2, causal, dtype):
    """The reference dispatches the operator over float32 and float64 too
    (attention_kernel.cu:269-281); here such q, k, v keep their storage and
    arithmetic: y, w and the three gradients within 1e-4 (float32) / 1e-12
    (float64) of the oracle, and w holds exact zeros above the diagonal."""
    _run(B, L1, L2, NH, H1, H2, causal, dtype, seed=L1 + 2 * L2, scale=0.8)
    if causal:
        g = torch.Generator().manual_seed(1)
        q = torch.randn(B, L1, NH, H1, generator=g).to(dtype).cuda()
        k = torch.randn(B, L2, NH, H1, generator=g).to(dtype).cuda()
        v = torch.randn(B, L2, NH, H2, generator=g).to(dtype).cuda()
        _, w = ops.attention_fwd(q, k, v, 1.0, 0.0, True)
        assert torch.count_nonzero(torch.triu(w, diagonal=L2 - L1 + 1)) == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,L1,L2,NH,H1,H2,causal", [
    (2, 768, 768, 2, 256, 512, True),     # three row blocks, two slabs per key tile
    (1, 700, 1000, 2, 128, 64, True),     # ragged rows, prefix of 300 keys, key count not a multiple of 64
    (3, 333, 1336, 1, 64, 72, True),      # one slab per key tile, long prefix
    (1, 520, 520, 3, 64, 128, False),     # every row sees every key
    (1, 1, 264, 2, 256, 256, False),      # one new token on a cache
    (9, 256, 256, 1, 128, 256, True),     # a (batch, head) count that is no multiple of the XCD count
    (2, 1100, 1100, 4, 256, 64, True),    # five row blocks, the last one ragged
])
def test_scores_and_softmax_in_one_kernel(B, L1, L2, NH, H1, H2, causal, dtype):
    """Head widths of 64, 128 and 256 with a key count that is a multiple of 8 compute the scores
    and their softmax in one kernel (two passes over the key tiles, nothing but P written):
    probabilities, values and all gradients against the float64 oracle."""
    _run(B, L1, L2, NH, H1, H2, causal, dtype, seed=L1 + L2 + H1)


@pytest.mark.parametrize("B,L1,L2,NH,H1,H2,causal", [
    (1, 8, 8, 1, 64, 64, True),           # fewer keys than one slab holds
    (2, 5, 40, 1, 128, 32, True),         # five new rows on a prefix of 35 keys
    (1, 24, 24, 2, 256, 8, False),
    (3, 1, 8, 1, 64, 16, False),          # one row, eight keys
])
def test_one_kernel_scores_on_tiny_shapes(B, L1, L2, NH, H1, H2, causal):
    _run(B, L1, L2, NH, H1, H2, causal, torch.bfloat16, seed=3 * L1 + L2)


def test_one_kernel_scores_with_large_logits():
    """Scores of several hundred in magnitude: the exponentials are taken relative to the row maximum
    (in both passes), so rows whose probabilities are all but one-hot come out exact and nothing
    overflows; compared with the float64 oracle on the same bf16 inputs."""
    g = torch.Generator().manual_seed(5)
    B, L, NH, H1, H2 = 1, 320, 2, 128, 64
    q = (6 * torch.randn(B, L, NH, H1, generator=g)).bfloat16()
    k = (6 * torch.randn(B, L, NH, H1, generator=g)).bfloat16()
    v = torch.randn(B, L, NH, H2, generator=g).bfloat16()
    y, w = ops.attention_fwd(q.cuda(), k.cuda(), v.cuda(), 1.0, 0.0, True)
    wy, ww = oa.chunk_attention_fwd(q, k, v, 1.0, True)
    assert torch.isfinite(w.float()).all() and torch.isfinite(y.float()).all()
    assert rel_err(w, ww) <= TOL and rel_err(y, wy) <= TOL
    assert torch.allclose(w.float().sum(-1).cpu(), torch.ones(B, NH, L), atol=2e-2)


def test_random_shapes():
    """Seeded random shapes with a key count that is a multiple of 64: ragged query counts,
    key/value prefixes of any length, causal and not, any head width that is a multiple of 8."""
    import random
    rnd = random.Random(6464)
    for case in range(12):
        L2 = 64 * rnd.randint(1, 20)
        L1 = rnd.choice([L2, rnd.randint(1, L2), max(1, L2 - 64 * rnd.randint(0, 3))])
        B, NH = rnd.randint(1, 2), rnd.randint(1, 3)
        H1, H2 = rnd.choice([8 * rnd.randint(1, 12), 64, 128]), 8 * rnd.randint(1, 40)
        causal = rnd.random() < 0.7
        _run(B, L1, L2, NH, H1, H2, causal, torch.bfloat16, seed=case, scale=0.7)


def test_causal_with_fewer_keys_than_queries_fails_loudly():
    q = torch.zeros(1, 8, 1, 16, dtype=torch.bfloat16, device="cuda")
    k = torch.zeros(1, 4, 1, 16, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="L2 >= L1"):
        ops.attention_fwd(q, k, k.clone(), 1.0, 0.0, True)


@pytest.mark.parametrize("B,L1,L2,NH,H1,H2", [(2, 1, 77, 2, 32, 64), (1, 130, 260, 1, 64, 64)])
def test_non_causal_rectangular(B, L1, L2, NH, H1, H2):
    _run(B, L1, L2, NH, H1, H2, False, torch.bfloat16, seed=7, scale=0.5)


def test_config3_shape_one_chunk():
    """BASELINE config 3 shape (chunk 4096, 4 heads, qk 256, value 2048), one chunk."""
    io = synthetic.attention_inputs(1, 4096, 4, 256, 2048, 1003)
    y, w = ops.attention_fwd(io["q"].cuda(), io["k"].cuda(), io["v"].cuda(), 1.0, 0.0, True)
    wy, _ = oa.chunk_attention_fwd(io["q"], io["k"], io["v"], 1.0, True)
    assert rel_err(y, wy) <= TOL
    dq, dk, dv = ops.attention_bwd(io["dy"].cuda(), io["q"].cuda(), io["k"].cuda(), io["v"].cuda(), w, 1.0, True)
    wdq, wdk, wdv = oa.chunk_attention_bwd(io["dy"], io["q"], io["k"], io["v"], 1.0, True)
    assert rel_err(dq, wdq) <= TOL and rel_err(dk, wdk) <= TOL and rel_err(dv, wdv) <= TOL


def test_full_config3_properties():
    """Size-independent checks on all 8 chunks x 4 heads of config 3: chunks are
    independent (a permutation of chunks permutes the output), row 0 of every
    chunk returns v[0], and y stays inside the convex hull of the values."""
    io = synthetic.attention_inputs(8, 4096, 4, 256, 2048, 1003)
    q, k, v = io["q"].cuda(), io["k"].cuda(), io["v"].cuda()
    y, _ = ops.attention_fwd(q, k, v, 1.0, 0.0, True)
    perm = torch.tensor([3, 0, 7, 1, 6, 2, 5, 4], device="cuda")
    yp, _ = ops.attention_fwd(q[perm].contiguous(), k[perm].contiguous(), v[perm].contiguous(), 1.0, 0.0, True)
    assert torch.equal(yp, y[perm])
    assert rel_err(y[:, 0], v[:, 0]) <= 1e-2
    assert y.float().abs().max() <= v.float().abs().max() * 1.01


def test_autograd_function_and_module():
    torch.manual_seed(0)
    bs, slen, NH, zd, vd, chunk = 2, 512, 2, 32, 64, 256
    attn = _InnerAttention(zd, vd, NH, chunk, 0.0, "fused").cuda()
    g = torch.Generator().manual_seed(3)
    xq = (torch.randn(bs, slen, NH * zd, generator=g) / zd ** 0.5).bfloat16()
    xk = (torch.randn(bs, slen, NH * zd, generator=g) / zd ** 0.5).bfloat16()
    xv = torch.randn(bs, slen, NH * vd, generator=g).bfloat16()
    dy = torch.randn(bs, slen, NH * vd, generator=g).bfloat16()
    cq, ck, cv = [t.cuda().requires_grad_(True) for t in (xq, xk, xv)]
    out, cache = attn(cq, ck, cv, None, None)
    assert cache is None and out.shape == (bs, slen, NH * vd)
    out.backward(dy.cuda())
    nc = slen // chunk
    oq = xq.view(bs * nc, chunk, NH, zd)
    okk = xk.view(bs * nc, chunk, NH, zd)
    ov = xv.view(bs * nc, chunk, NH, vd)
    wy, _ = oa.chunk_attention_fwd(oq, okk, ov, 1.0, True)
    assert rel_err(out, wy.reshape(bs, slen, -1)) <= TOL
    wdq, wdk, wdv = oa.chunk_attention_bwd(dy.view(bs * nc, chunk, NH, vd), oq, okk, ov, 1.0, True)
    assert rel_err(cq.grad, wdq.reshape(bs, slen, -1)) <= TOL
    assert rel_err(ck.grad, wdk.reshape(bs, slen, -1)) <= TOL
    assert rel_err(cv.grad, wdv.reshape(bs, slen, -1)) <= TOL


def test_unsupported_cases_fail_loudly():
    q = torch.zeros(1, 8, 1, 8, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match=r"\[0, 1\]"):
        ops.attention_fwd(q, q, q, 1.0, 1.5, True)   # not a probability
    with pytest.raises(RuntimeError, match="complex64"):
        ops.attention_fwd(q.to(torch.complex64), q.to(torch.complex64), q.to(torch.complex64), 1.0, 0.0, True)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32, torch.float64])
@pytest.mark.parametrize("shape,causal", [
    ((2, 3, 300, 300), True), ((1, 2, 100, 260), True), ((4, 64, 512), False), ((1, 1, 1, 40), True),
    ((2, 1, 50, 4100), False),   # rows longer than the register-resident kernels take
])
def test_standalone_softmax(shape, causal, dtype):
    """attention_softmax_fwd/bwd against float64: y = softmax over the last
    axis with the bottom-right aligned causal mask, zeros above it;
    dx = y o (dy - sum(y o dy))."""
    from megalodon_amd.fused_ops import attention_softmax
    g = torch.Generator().manual_seed(sum(shape))
    x = (2.0 * torch.randn(*shape, generator=g)).to(dtype)
    dy = torch.randn(*shape, generator=g).to(dtype)
    L1, L2 = shape[-2], shape[-1]
    xd = x.clone().double().requires_grad_(True)   # its own leaf, also when x is float64 already
    if causal:
        r = torch.arange(L1).view(L1, 1)
        c = torch.arange(L2).view(1, L2)
        want = torch.softmax(xd.masked_fill(c > r + (L2 - L1), float("-inf")), dim=-1)
    else:
        want = torch.softmax(xd, dim=-1)
    want.backward(dy.double())
    xg = x.cuda().requires_grad_(True)
    y = attention_softmax(xg, 0.0, causal, True)
    tol = {torch.float32: TOL_F32, torch.float64: TOL_F64}.get(dtype, TOL)
    assert y.dtype == dtype and y.shape == x.shape
    assert rel_err(y, want.detach()) <= tol
    if causal:
        assert torch.count_nonzero(torch.triu(y.float(), diagonal=L2 - L1 + 1)) == 0
    y.backward(dy.cuda())
    assert rel_err(xg.grad, xd.grad) <= tol


@pytest.mark.parametrize("causal", [True, False])
def test_swift_attention_module_matches_oracle(causal):
    """SwiftAttention (the reference's fused_attention.py module) forward and
    backward, bf16, against the float64 oracle; eval mode ignores its dropout."""
    from megalodon_amd.modules import SwiftAttention
    B, L, N, H1, H2 = 2, 300, 2, 64, 128
    g = torch.Generator().manual_seed(11)
    q, k = (torch.randn(B, L, N, H1, generator=g).bfloat16() / H1 ** 0.25 for _ in range(2))
    v = torch.randn(B, L, N, H2, generator=g).bfloat16()
    dy = torch.randn(B, L, N, H2, generator=g).bfloat16()
    m = SwiftAttention(scale=0.5, dropout=0.3, use_causal_mask=causal).eval()
    assert "dropout=0.3" in repr(m) and f"causal={causal}" in repr(m)
    qc, kc, vc = (t.cuda().requires_grad_(True) for t in (q, k, v))
    y = m(qc, kc, vc)
    y.backward(dy.cuda())
    want, _ = oa.chunk_attention_fwd(q, k, v, 0.5, causal)
    wq, wk, wv = oa.chunk_attention_bwd(dy, q, k, v, 0.5, causal)
    assert rel_err(y, want) <= 2e-2
    assert rel_err(qc.grad, wq) <= 2e-2 and rel_err(kc.grad, wk) <= 2e-2 and rel_err(vc.grad, wv) <= 2e-2


@pytest.mark.parametrize("causal", [True, False])
def test_attention_softmax_module_matches_torch(causal):
    """AttentionSoftmax (the reference's attention_softmax.py module) in eval
    mode: rows of softmax with the bottom-right aligned causal mask, and the
    gradient of a float64 softmax."""
    from megalodon_amd.modules import AttentionSoftmax
    B, N, L1, L2 = 2, 3, 70, 100
    g = torch.Generator().manual_seed(12)
    x = torch.randn(B, N, L1, L2, generator=g).bfloat16()   # the op takes 16-bit scores
    dy = torch.randn(B, N, L1, L2, generator=g).bfloat16()
    m = AttentionSoftmax(dropout=0.5, use_causal_mask=causal).eval()
    xc = x.cuda().requires_grad_(True)
    y = m(xc)
    y.backward(dy.cuda())
    x64 = x.double().requires_grad_(True)
    s = x64
    if causal:
        r = torch.arange(L1).view(L1, 1)
        c = torch.arange(L2).view(1, L2)
        s = x64.masked_fill(c > r + (L2 - L1), float("-inf"))
    want = torch.softmax(s, dim=-1)
    want.backward(dy.double())
    assert rel_err(y, want.detach()) <= 2e-2
    assert rel_err(xc.grad, x64.grad) <= 2e-2
