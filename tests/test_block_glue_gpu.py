"""The block's glue kernels: tiled transpose (bit-exact, a byte move) and the
SiLU gates against float64 (`silu(a) * b` and its autograd gradient):
rel err <= 1e-4 float32, <= 2e-2 bfloat16 / float16."""
import pytest
import torch
import torch.nn.functional as F

from conftest import rel_err
from megalodon_amd import extension as ops
from megalodon_amd.fused_ops import silu_mul, transpose_last2

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [
    (2, 256, 384),      # whole 128 x 128 tiles
    (1, 1000, 72),      # partial tiles on both sides, still 16-byte rows
    (3, 50, 77),        # ragged: element-wise path
    (2, 3, 8, 4096),    # leading dimensions fold into the batch; R far below a tile
    (1, 1, 1),
])
def test_transpose_is_a_bit_exact_move(shape, dtype):
    g = torch.Generator().manual_seed(sum(shape))
    x = torch.randn(*shape, generator=g).to(dtype).cuda()
    y = ops.transpose_last2(x)
    assert y.is_contiguous() and y.shape == x.transpose(-2, -1).shape
    assert torch.equal(y, x.transpose(-2, -1).contiguous())
    assert torch.equal(ops.transpose_last2(y), x)


def test_transpose_of_views_and_unaligned_buffers():
    base = torch.randn(2 * 64 * 128 + 1, device="cuda").bfloat16()
    x = base[1:].view(2, 64, 128)                 # 2-byte aligned only
    assert torch.equal(ops.transpose_last2(x), x.transpose(1, 2).contiguous())
    v = torch.randn(4, 128, 256, device="cuda").half()[:, :, ::2]   # strided input
    assert torch.equal(ops.transpose_last2(v), v.transpose(1, 2).contiguous())
    e = torch.empty(0, 8, 16, device="cuda", dtype=torch.bfloat16)
    assert ops.transpose_last2(e).shape == (0, 16, 8)


def test_transpose_autograd_and_full_size():
    x = torch.randn(2, 96, 160, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    w = torch.randn(2, 160, 96, device="cuda", dtype=torch.bfloat16)
    (transpose_last2(x) * w).sum().backward()
    assert torch.equal(x.grad, w.transpose(1, 2))
    # config-4 activation: (1, 32768, 4096) both ways
    big = torch.randn(1, 32768, 4096, device="cuda").bfloat16()
    t = ops.transpose_last2(big)
    assert torch.equal(t, big.transpose(1, 2).contiguous()) and torch.equal(ops.transpose_last2(t), big)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 2e-2), (torch.float16, 2e-2)])
@pytest.mark.parametrize("shape", [(4, 300, 64), (1003,), (2, 7, 9), (8,)])
def test_silu_gate_matches_float64(shape, dtype, tol):
    g = torch.Generator().manual_seed(len(shape) + shape[0])
    a = (torch.randn(*shape, generator=g) * 3).to(dtype)
    b = torch.randn(*shape, generator=g).to(dtype)
    dy = torch.randn(*shape, generator=g).to(dtype)
    ag, bg = a.cuda().requires_grad_(True), b.cuda().requires_grad_(True)
    y = silu_mul(ag, bg)
    y.backward(dy.cuda())
    a64, b64 = a.double().requires_grad_(True), b.double().requires_grad_(True)
    want = F.silu(a64) * b64
    want.backward(dy.double())
    assert y.dtype == dtype and rel_err(y, want) <= tol
    assert rel_err(ag.grad, a64.grad) <= tol and rel_err(bg.grad, b64.grad) <= tol


def test_silu_gate_edge_values_and_unaligned():
    a = torch.tensor([0.0, -100.0, 100.0, -20.0, 20.0, 1e-3, -1e-3, 88.0, -88.0], device="cuda")
    b = torch.full_like(a, 2.0)
    y = ops.silu_mul_fwd(a, b)
    want = (F.silu(a.double()) * 2.0)
    assert torch.isfinite(y).all() and rel_err(y, want) <= 1e-5
    da, db = ops.silu_mul_bwd(torch.ones_like(a), a, b)
    assert torch.isfinite(da).all() and torch.isfinite(db).all()
    base = torch.randn(4097, device="cuda").bfloat16()
    u, v = base[1:], base[:-1].clone()
    assert rel_err(ops.silu_mul_fwd(u, v), F.silu(u.double()) * v.double()) <= 2e-2
    with pytest.raises(RuntimeError, match="same shape"):
        ops.silu_mul_fwd(u, v[:-1])


def test_silu_gate_at_the_feed_forward_size():
    # (32768, 11008) bfloat16 as in config 4: compare a strided sample with float64
    n = 32768 * 11008
    a = torch.randn(n, device="cuda", dtype=torch.bfloat16)
    b = torch.randn(n, device="cuda", dtype=torch.bfloat16)
    y = ops.silu_mul_fwd(a, b)
    idx = torch.arange(0, n, 4099, device="cuda")
    assert rel_err(y[idx], F.silu(a[idx].double()) * b[idx].double()) <= 2e-2
    assert rel_err(y[-70000:], F.silu(a[-70000:].double()) * b[-70000:].double()) <= 2e-2
    da, db = ops.silu_mul_bwd(y, a, b)
    s = torch.sigmoid(a[idx].double())
    assert rel_err(db[idx], y[idx].double() * a[idx].double() * s) <= 2e-2
    assert rel_err(da[idx], y[idx].double() * b[idx].double() * s * (1 + a[idx].double() * (1 - s))) <= 2e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape,out,bias", [((2, 300, 256), 512, True), ((640, 1024), 264, False), ((3, 5, 7, 64), 72, True),
                                            # layers of a whole 256 x 256 tile per compute unit: the weight gradient
                                            # runs on the attention operator's product kernel
                                            ((1, 8192, 2048), 8192, True), ((4128, 8192), 2048, False), ((4100, 4096), 4096, False)])
def test_linear_with_transposed_weight_backward_matches_float64(shape, out, bias, dtype):
    from megalodon_amd.modules.linear import Linear
    torch.manual_seed(out)
    lin = Linear(shape[-1], out, bias=bias).cuda().to(dtype)
    x = torch.randn(*shape, device="cuda").to(dtype).requires_grad_(True)
    dy = torch.randn(*shape[:-1], out, device="cuda").to(dtype)
    y = lin(x)
    y.backward(dy)
    x64 = x.detach().double().requires_grad_(True)
    w64 = lin.weight.detach().double().requires_grad_(True)
    b64 = lin.bias.detach().double().requires_grad_(True) if bias else None
    want = F.linear(x64, w64, b64)
    want.backward(dy.double())
    assert rel_err(y, want) <= 2e-2 and rel_err(x.grad, x64.grad) <= 2e-2
    assert rel_err(lin.weight.grad, w64.grad) <= 2e-2
    if bias:
        assert rel_err(lin.bias.grad, b64.grad) <= 2e-2
    # state dicts are those of nn.Linear; without gradients the module is F.linear itself
    ref = torch.nn.Linear(shape[-1], out, bias=bias).cuda().to(dtype)
    ref.load_state_dict(lin.state_dict())
    with torch.no_grad():
        assert torch.equal(lin(x), ref(x))


def test_random_shapes_sweep():
    """Forty seeded random shapes per kernel: transpose against PyTorch's own
    (bit-exact), the SiLU gate and the norms against float64 (2e-2, bfloat16)."""
    import random
    from megalodon_amd.fused_ops import layer_norm_plus_one
    rnd = random.Random(20240)
    for _ in range(40):
        Z, R, C = rnd.randint(1, 3), rnd.choice([8, 40, 129, 256, 264, 1000]), rnd.choice([8, 24, 130, 256, 520])
        x = torch.randn(Z, R, C, device="cuda").bfloat16()
        assert torch.equal(ops.transpose_last2(x), x.transpose(1, 2).contiguous()), (Z, R, C)
        n = rnd.randint(1, 5000)
        a, b = torch.randn(n, device="cuda").bfloat16(), torch.randn(n, device="cuda").bfloat16()
        assert rel_err(ops.silu_mul_fwd(a, b), F.silu(a.double()) * b.double()) <= 2e-2, n
        rows, D = rnd.randint(1, 70), rnd.choice([128, 256, 512, 1024, 2048, 4096, 96, 300, 1000])
        rms = rnd.random() < 0.5
        xx = (torch.randn(rows, D, device="cuda") + 0.3).bfloat16()
        w = (torch.randn(D, device="cuda") * 0.2).bfloat16()
        bb = None if rms else (torch.randn(D, device="cuda") * 0.2).bfloat16()
        y = layer_norm_plus_one(xx, w, bb, 1e-5, rms)
        x64 = xx.double()
        if rms:
            want = x64 * torch.rsqrt(x64.pow(2).mean(-1, keepdim=True) + 1e-5) * (w.double() + 1)
        else:
            want = F.layer_norm(x64, (D,), w.double() + 1, bb.double(), 1e-5)
        assert rel_err(y, want) <= 2e-2, (rows, D, rms)


def test_empty_inputs_are_accepted():
    from megalodon_amd.fused_ops import qk_norm_rotary
    e = torch.empty(0, device="cuda", dtype=torch.bfloat16)
    assert ops.silu_mul_fwd(e, e).numel() == 0
    da, db = ops.silu_mul_bwd(e, e, e)
    assert da.numel() == 0 and db.numel() == 0
    assert ops.dropout(e, 0.5, 1, 0).numel() == 0
    z = torch.empty(2, 0, 512, device="cuda", dtype=torch.bfloat16)
    g = torch.zeros(2, 512, device="cuda", dtype=torch.bfloat16)
    q, k = qk_norm_rotary(z, g, g, None, 64, 1e-5)
    assert q.shape == (2, 0, 512) and k.shape == (2, 0, 512)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("tokens,n_out,n_in", [(4096, 512, 768), (4128, 2304, 264), (64, 8, 8), (8200, 1000, 520),
                                               (4099, 130, 77)])   # the last: off the aligned path
def test_linear_weight_grad_matches_float64(tokens, n_out, n_in, dtype, monkeypatch):
    """dW = dy^T x on the attention product kernel against float64 (2e-2, 16-bit output of a
    float32 accumulation), for every band width of the tile order (identical bits: the order of
    the tiles does not enter a tile's sum)."""
    g = torch.Generator().manual_seed(tokens + n_out)
    dy = torch.randn(tokens, n_out, generator=g).to(dtype).cuda()
    x = torch.randn(tokens, n_in, generator=g).to(dtype).cuda()
    want = dy.double().t() @ x.double()
    got = ops.linear_weight_grad(dy, x)
    assert got.shape == (n_out, n_in) and got.dtype == dtype
    assert rel_err(got, want) <= 2e-2
    for ng in ("0", "3", "16"):
        monkeypatch.setenv("MEGA_GEMM_NGROUP", ng)
        assert torch.equal(ops.linear_weight_grad(dy, x), got)


def test_linear_group_matches_float64_and_separate_layers():
    """Layers that read one input (`linear_group`): outputs are those of the layers one by one,
    and the shared input gradient, accumulated inside the GEMM, and every parameter gradient
    match float64 (2e-2, bfloat16)."""
    from megalodon_amd.modules.linear import Linear, linear_group
    torch.manual_seed(3)
    layers = [Linear(256, 512, bias=True), Linear(256, 72, bias=False), Linear(256, 256, bias=True)]
    layers = [l.cuda().bfloat16() for l in layers]
    x = torch.randn(3, 100, 256, device="cuda").bfloat16().requires_grad_(True)
    dys = [torch.randn(3, 100, l.out_features, device="cuda").bfloat16() for l in layers]
    ys = linear_group(x, layers)
    with torch.no_grad():
        for y, l in zip(ys, layers):
            assert torch.equal(y, l(x))
    torch.autograd.backward(ys, dys)
    x64 = x.detach().double().requires_grad_(True)
    w64 = [l.weight.detach().double().requires_grad_(True) for l in layers]
    b64 = [None if l.bias is None else l.bias.detach().double().requires_grad_(True) for l in layers]
    torch.autograd.backward([F.linear(x64, w, b) for w, b in zip(w64, b64)], [d.double() for d in dys])
    assert rel_err(x.grad, x64.grad) <= 2e-2
    for l, w, b in zip(layers, w64, b64):
        assert rel_err(l.weight.grad, w.grad) <= 2e-2
        if b is not None:
            assert rel_err(l.bias.grad, b.grad) <= 2e-2
    # one output unused downstream: its gradient is taken as zero
    x.grad = None
    y0, _, _ = linear_group(x, layers)
    y0.backward(dys[0])
    x64.grad = None
    F.linear(x64, w64[0], b64[0]).backward(dys[0].double())
    assert rel_err(x.grad, x64.grad) <= 2e-2


def test_linear_with_residual_inside_the_gemm():
    from megalodon_amd.modules.linear import Linear
    torch.manual_seed(4)
    lin = Linear(256, 384, bias=False).cuda().bfloat16()
    x = torch.randn(3, 70, 256, device="cuda").bfloat16().requires_grad_(True)
    r = torch.randn(3, 70, 384, device="cuda").bfloat16().requires_grad_(True)
    dy = torch.randn(3, 70, 384, device="cuda").bfloat16()
    y = lin(x, residual=r)
    y.backward(dy)
    x64, r64 = x.detach().double().requires_grad_(True), r.detach().double().requires_grad_(True)
    w64 = lin.weight.detach().double().requires_grad_(True)
    want = F.linear(x64, w64) + r64
    want.backward(dy.double())
    assert rel_err(y, want) <= 2e-2 and rel_err(x.grad, x64.grad) <= 2e-2
    assert rel_err(lin.weight.grad, w64.grad) <= 2e-2 and torch.equal(r.grad, dy)
    with torch.no_grad():
        assert rel_err(lin(x, residual=r), want) <= 2e-2
    # a layer with bias keeps the separate add
    lb = Linear(256, 384, bias=True).cuda().bfloat16()
    assert rel_err(lb(x, residual=r), F.linear(x64, lb.weight.double(), lb.bias.double()) + r64) <= 2e-2


@pytest.mark.parametrize("nbytes", [16, 4096 + 16, 3 * 1024 * 1024 + 48])
@pytest.mark.parametrize("two", [False, True])
def test_stream_copy_reference_kernel(nbytes, two):
    from megalodon_amd import extension as ops
    a = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device="cuda")
    b = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device="cuda") if two else None
    for wgs in (1, 7, 512):
        for nt in (False, True):
            out = ops.stream_copy(a, b, wgs, nt)
            assert torch.equal(out, a ^ b if two else a)
