"""Pins oracle/block.py: its two helpers against library routines and explicit
formulas, and the wiring of `mega_block_forward` by special cases that a wrong
connection (v from the wrong tensor, a dropped residual, a missing 1/sqrt(Dh),
positions counted over the sequence instead of the chunk) would fail, plus an
independent restatement of the whole block from other primitives (a sequential
EMA recurrence instead of the FFT, scaled_dot_product_attention per chunk,
F.rms_norm, brute-force prefix statistics)."""
import math

import torch
import torch.nn.functional as F

from oracle import block as ob
from oracle import cema as ocema
from oracle import timestep_norm as otn

CFG = dict(num_heads=2, ndim=4, chunk_size=8, groups=2)
D, Z, H, FF = 8, 8, 12, 10


def _params(seed=0, D=D, Z=Z, H=H, FF=FF, ndim=4):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64) * 0.5
    return {
        "mega.timenorm.weight": r(D) * 0.2, "mega.timenorm.bias": r(D) * 0.2,
        "mega.cema.alpha": r(D, ndim, 1), "mega.cema.delta": r(D, ndim, 1), "mega.cema.theta": r(D, 1, 1),
        "mega.cema.gamma": r(D, ndim, 2), "mega.cema.omega": r(D, 1),
        "mega.rmsnorm.weight": r(D) * 0.2,
        "mega.wz.weight": r(Z, D), "mega.wz.bias": r(Z),
        "mega.wv.weight": r(H, D), "mega.wv.bias": r(H),
        "mega.wr.weight": r(H, D), "mega.wr.bias": r(H),
        "mega.wh1.weight": r(D, D), "mega.wh1.bias": r(D),
        "mega.wh2.weight": r(D, H),
        "mega.gamma": r(2, Z) * 0.3, "mega.beta": r(2, Z) * 0.3,
        "nffn.norm.weight": r(D) * 0.2, "nffn.norm.bias": r(D) * 0.2,
        "nffn.fc1.weight": r(FF, D), "nffn.fc2.weight": r(D, FF), "nffn.fc3.weight": r(FF, D),
    }


def _x(B=2, L=24, seed=1):
    return torch.randn(B, L, D, generator=torch.Generator().manual_seed(seed), dtype=torch.float64)


def _freqs(C, Dh, base=10000.0):
    inv = 1.0 / (base ** (torch.arange(0, Dh, 2, dtype=torch.float64) / Dh))
    ang = torch.outer(torch.arange(C, dtype=torch.float64), inv)
    return torch.polar(torch.ones_like(ang), ang)


def test_rms_matches_library_rms_norm():
    x = _x()
    w = torch.randn(D, dtype=torch.float64)
    assert torch.allclose(ob._rms(x, w, 1e-5), F.rms_norm(x, (D,), w + 1.0, 1e-5), atol=1e-14)
    assert torch.allclose(ob._rms(x, None, 1e-3), F.rms_norm(x, (D,), None, 1e-3), atol=1e-14)
    # textbook special case: a constant row of value c maps to c / sqrt(c^2 + eps)
    c = torch.full((1, 1, D), 3.0, dtype=torch.float64)
    assert torch.allclose(ob._rms(c, None, 0.25), c / math.sqrt(9.25), atol=1e-15)


def test_rotary_is_the_pairwise_plane_rotation():
    # rotary_positional_embedding.py:53-77: elements (2i, 2i+1) rotate by the angle of freqs_cis[pos, i]
    C, heads, Dh = 5, 3, 6
    x = torch.randn(2, C, heads, Dh, generator=torch.Generator().manual_seed(3), dtype=torch.float64)
    fc = _freqs(C, Dh)
    got = ob.rotary(x, fc)
    ang = fc.angle()
    for pos in range(C):
        for i in range(Dh // 2):
            c, s = math.cos(ang[pos, i]), math.sin(ang[pos, i])
            a, b = x[:, pos, :, 2 * i], x[:, pos, :, 2 * i + 1]
            assert torch.allclose(got[:, pos, :, 2 * i], a * c - b * s, atol=1e-14)
            assert torch.allclose(got[:, pos, :, 2 * i + 1], a * s + b * c, atol=1e-14)
    # position 0 is the identity; norms of pairs are kept
    assert torch.allclose(got[:, 0], x[:, 0], atol=1e-15)
    assert torch.allclose(got.pow(2).sum(-1), x.pow(2).sum(-1), atol=1e-12)


def test_zero_fc2_returns_the_block_input():
    p = _params()
    p["nffn.fc2.weight"] = torch.zeros_like(p["nffn.fc2.weight"])
    x = _x()
    assert torch.equal(ob.mega_block_forward(p, x, **CFG), x)


def test_zero_output_projections_leave_ffn_of_input():
    # wh1 = wh2 = 0 (and no bias): the attention sub-layer returns x, so the block
    # is x + fc2(silu(fc1 n) * fc3 n) with n = LayerNorm(x) (weight + 1), and the
    # FFN's residual is the block input (model/mega.py:86-88)
    p = _params()
    for k in ("mega.wh1.weight", "mega.wh1.bias", "mega.wh2.weight"):
        p[k] = torch.zeros_like(p[k])
    x = _x()
    mu, var = x.mean(-1, keepdim=True), x.var(-1, unbiased=False, keepdim=True)
    n = (x - mu) / torch.sqrt(var + 1e-5) * (p["nffn.norm.weight"] + 1.0) + p["nffn.norm.bias"]
    a, b = n @ p["nffn.fc1.weight"].T, n @ p["nffn.fc3.weight"].T
    want = (a * torch.sigmoid(a) * b) @ p["nffn.fc2.weight"].T + x
    assert torch.allclose(ob.mega_block_forward(p, x, **CFG), want, atol=1e-12)


def test_causal_and_chunk_local():
    p = _params()
    x = _x(B=1, L=24)
    base = ob.mega_block_forward(p, x, **CFG)
    x2 = x.clone()
    x2[0, 13] += 1.0
    moved = ob.mega_block_forward(p, x2, **CFG)
    # no earlier output moves (the FFT and the prefix sums leave rounding noise only)
    assert (moved[0, :13] - base[0, :13]).abs().max() < 1e-11
    # every later token does (EMA state and running statistics carry the change forward)
    assert (moved[0, 13:] - base[0, 13:]).abs().amax(dim=-1).min() > 1e-6


def test_value_path_reads_timestep_norm_output_and_gate_reads_mx():
    # rmsnorm.weight = -1 makes mx = 0: q, k become position-independent, so the
    # softmax is the uniform average over the keys of the chunk so far, the gate
    # is silu(wr.bias) and wh1 contributes its bias only.  v must still follow
    # out_tsn (moving_average_gated_attention.py:327: wv takes out_tsn, not mx).
    p = _params()
    p["mega.rmsnorm.weight"] = torch.full_like(p["mega.rmsnorm.weight"], -1.0)
    x = _x(B=2, L=24)

    B, L, _ = x.shape
    C = CFG["chunk_size"]
    pc, pm, pv = torch.zeros(B, dtype=torch.int64), torch.zeros(B, 2, dtype=torch.float64), torch.ones(B, 2, dtype=torch.float64)
    out_tsn = otn.group_timestep_norm_fwd(x, pc, pm, pv, p["mega.timenorm.weight"] + 1.0, p["mega.timenorm.bias"],
                                          None, 2, 1e-5)[0]
    v = F.silu(out_tsn @ p["mega.wv.weight"].T + p["mega.wv.bias"]).view(B, L // C, C, -1)
    steps = torch.arange(1, C + 1, dtype=torch.float64).view(1, 1, C, 1)
    avg = (v.cumsum(2) / steps).reshape(B, L, -1)
    gate = F.silu(p["mega.wr.bias"])
    y1 = p["mega.wh1.bias"] + (avg * gate) @ p["mega.wh2.weight"].T + x
    n = F.layer_norm(y1, (D,), p["nffn.norm.weight"] + 1.0, p["nffn.norm.bias"], 1e-5)
    want = (F.silu(n @ p["nffn.fc1.weight"].T) * (n @ p["nffn.fc3.weight"].T)) @ p["nffn.fc2.weight"].T + x
    assert torch.allclose(ob.mega_block_forward(p, x, **CFG), want, atol=1e-11)


def _restated_block(p, x, num_heads, ndim, chunk_size, groups, freqs_cis=None, eps=1e-5):
    """The block from other primitives: prefix statistics by brute force, the EMA
    as its recurrence, library rms_norm / layer_norm / scaled_dot_product_attention."""
    B, L, Dm = x.shape
    Dg = Dm // groups
    xg = x.view(B, L, groups, Dg)
    out_tsn = torch.empty_like(xg)
    for t in range(L):
        seen = xg[:, :t + 1]                                   # prior count 0: the prior is ignored
        mu = seen.mean(-1).mean(1)                             # mean of per-step means
        ex2 = (seen * seen).mean(-1).mean(1)
        var = ex2 - mu * mu
        out_tsn[:, t] = (xg[:, t] - mu.unsqueeze(-1)) / torch.sqrt(var.unsqueeze(-1) + eps)
    out_tsn = out_tsn.view(B, L, Dm) * (p["mega.timenorm.weight"] + 1.0) + p["mega.timenorm.bias"]
    # CEMA as a recurrence (complex_exponential_moving_average.py:100-117 for the coefficients)
    pp = torch.sigmoid(p["mega.cema.alpha"]).squeeze(-1)
    rad = 1.0 - pp * torch.sigmoid(p["mega.cema.delta"]).squeeze(-1)
    ang = torch.sigmoid(p["mega.cema.theta"]).view(Dm, 1) * (2 * math.pi / ndim) * torch.arange(1, ndim + 1, dtype=torch.float64)
    q = torch.polar(rad, ang)
    gam = torch.view_as_complex(p["mega.cema.gamma"].contiguous()) * math.sqrt(1.0 / ndim)
    h = torch.zeros(B, Dm, ndim, dtype=torch.complex128)
    out_cema = torch.empty(B, L, Dm, dtype=torch.float64)
    for t in range(L):
        h = q * h + pp * out_tsn[:, t].unsqueeze(-1)
        out_cema[:, t] = (gam * h).sum(-1).real + out_tsn[:, t] * p["mega.cema.omega"].view(Dm)
    mx = F.rms_norm(out_cema, (Dm,), p["mega.rmsnorm.weight"] + 1.0, eps)
    zdim = p["mega.wz.weight"].shape[0]
    zh = zdim // num_heads
    z = (mx @ p["mega.wz.weight"].T + p["mega.wz.bias"]).view(B, L, num_heads, zh)
    z = F.rms_norm(z, (zh,), None, eps).view(B, L, zdim)
    qv = z * (p["mega.gamma"][0] + 1.0) / math.sqrt(zh) + p["mega.beta"][0]
    kv = z * (p["mega.gamma"][1] + 1.0) / math.sqrt(zh) + p["mega.beta"][1]
    v = F.silu(out_tsn @ p["mega.wv.weight"].T + p["mega.wv.bias"])
    r = F.silu(mx @ p["mega.wr.weight"].T + p["mega.wr.bias"])
    vh = v.shape[-1] // num_heads
    attn = torch.empty_like(v)
    for c0 in range(0, L, chunk_size):
        sl = slice(c0, c0 + chunk_size)
        qc = qv[:, sl].view(B, -1, num_heads, zh)
        kc = kv[:, sl].view(B, -1, num_heads, zh)
        if freqs_cis is not None:
            def rot(t):
                a, b = t[..., 0::2], t[..., 1::2]
                co, si = freqs_cis.real.unsqueeze(1), freqs_cis.imag.unsqueeze(1)
                return torch.stack((a * co - b * si, a * si + b * co), dim=-1).flatten(-2)
            qc, kc = rot(qc), rot(kc)
        vc = v[:, sl].view(B, -1, num_heads, vh)
        o = F.scaled_dot_product_attention(qc.transpose(1, 2), kc.transpose(1, 2), vc.transpose(1, 2),
                                           is_causal=True, scale=1.0)
        attn[:, sl] = o.transpose(1, 2).reshape(B, -1, num_heads * vh)
    y1 = mx @ p["mega.wh1.weight"].T + p["mega.wh1.bias"] + (attn * r) @ p["mega.wh2.weight"].T + x
    n = F.layer_norm(y1, (Dm,), p["nffn.norm.weight"] + 1.0, p["nffn.norm.bias"], eps)
    hid = F.silu(n @ p["nffn.fc1.weight"].T) * (n @ p["nffn.fc3.weight"].T)
    return hid @ p["nffn.fc2.weight"].T + x


def test_whole_block_against_independent_restatement():
    p = _params(seed=5)
    x = _x(B=2, L=24, seed=6)
    for fc in (None, _freqs(CFG["chunk_size"], Z // CFG["num_heads"])):
        got = ob.mega_block_forward(p, x, freqs_cis=fc, **CFG)
        want = _restated_block(p, x, freqs_cis=fc, **CFG)
        assert torch.allclose(got, want, atol=1e-10, rtol=1e-10)


def test_gradients_of_the_oracle_match_the_restatement():
    p = {k: v.requires_grad_(True) for k, v in _params(seed=7).items()}
    x = _x(B=1, L=16, seed=8).requires_grad_(True)
    dy = torch.randn(1, 16, D, generator=torch.Generator().manual_seed(2), dtype=torch.float64)
    names = sorted(p)
    g1 = torch.autograd.grad((ob.mega_block_forward(p, x, **CFG) * dy).sum(), [x] + [p[n] for n in names])
    g2 = torch.autograd.grad((_restated_block(p, x, **CFG) * dy).sum(), [x] + [p[n] for n in names])
    for n, a, b in zip(["x"] + names, g1, g2):
        assert torch.allclose(a, b, atol=1e-9, rtol=1e-8), n
