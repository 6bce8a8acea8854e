"""Oracle for one Megalodon block (float64 composition of the other oracles).

Follows megalodon/modules/moving_average_gated_attention.py:275-348,
megalodon/modules/normalized_feedforward_network.py:75-94,
megalodon/model/mega.py:79-88 and the `weight + 1` norm convention of
megalodon/modules/layer_norm.py:31,59.  `p` maps the parameter names of
`megalodon_amd.modules.MegaBlock.named_parameters()` to float64 tensors.

Test infrastructure only.  Pinned by tests/test_oracle_block.py: `_rms` against
torch.nn.functional.rms_norm, `rotary` against explicit plane rotations, the
wiring by special cases that a mis-routed tensor fails (zero fc2, zero wh1 /
wh2, rmsnorm weight -1, causality) and the whole block with all gradients by an
independent restatement from other primitives (EMA recurrence,
scaled_dot_product_attention, brute-force prefix statistics).
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F

from . import attention as oattn
from . import cema as ocema
from . import fftconv as offt
from . import timestep_norm as otn


def _rms(x, weight, eps):
    y = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * (weight + 1.0)


def rotary(x, freqs_cis):
    """x (B', C, heads, Dh), freqs_cis (C, Dh / 2) complex: neighbouring elements
    (2i, 2i+1) form a complex number that is multiplied by freqs_cis[position, i]
    (megalodon/modules/rotary_positional_embedding.py:53-77)."""
    xc = torch.view_as_complex(x.double().reshape(*x.shape[:-1], -1, 2))
    out = xc * freqs_cis.to(torch.complex128).unsqueeze(1)
    return torch.view_as_real(out).flatten(3)


def mega_block_forward(p, x, *, num_heads, ndim, chunk_size, groups, eps=1e-5, swiglu=True, freqs_cis=None):
    B, L, D = x.shape
    x = x.double()
    # TimestepNorm (prior count 0: buffers, not parameters)
    pc = torch.zeros(B, dtype=torch.int64)
    pm = torch.zeros(B, groups, dtype=torch.float64)
    pv = torch.ones(B, groups, dtype=torch.float64)
    out_tsn, _, _ = otn.group_timestep_norm_closed_form(
        x, pc, pm, pv, p["mega.timenorm.weight"] + 1.0, p["mega.timenorm.bias"], None, groups, eps)
    # CEMA
    pp, q, g = ocema.calc_coeffs(p["mega.cema.alpha"], p["mega.cema.delta"], p["mega.cema.theta"],
                                 p["mega.cema.gamma"], ndim)
    k = ocema.ema_weight_fwd(pp, q.log(), g, L)
    xt = out_tsn.transpose(1, 2)
    out_cema = (offt.fftconv_fwd(xt, k) + xt * p["mega.cema.omega"]).transpose(1, 2)
    mx = _rms(out_cema, p["mega.rmsnorm.weight"], eps)
    zdim = p["mega.wz.weight"].shape[0]
    zh = zdim // num_heads
    z = F.linear(mx, p["mega.wz.weight"], p["mega.wz.bias"]).view(B, L, num_heads, zh)
    z = _rms(z, None, eps).view(B, L, -1)
    gamma = (p["mega.gamma"] + 1.0) / math.sqrt(zh)
    z = z.unsqueeze(2) * gamma + p["mega.beta"]
    qq, kk = torch.unbind(z, dim=2)
    v = F.silu(F.linear(out_tsn, p["mega.wv.weight"], p["mega.wv.bias"]))
    r = F.silu(F.linear(mx, p["mega.wr.weight"], p["mega.wr.bias"]))
    hdim = v.shape[-1]
    vh = hdim // num_heads
    nc = max(1, L // chunk_size)
    C = L // nc
    qq, kk = qq.reshape(B * nc, C, num_heads, zh), kk.reshape(B * nc, C, num_heads, zh)
    if freqs_cis is not None:
        # position = index inside the chunk (moving_average_gated_attention.py:88-90,113-114)
        qq, kk = rotary(qq, freqs_cis), rotary(kk, freqs_cis)
    y, _ = oattn.chunk_attention_fwd(qq, kk, v.reshape(B * nc, C, num_heads, vh), 1.0, True)
    attn = y.reshape(B, L, hdim) * r
    h = F.linear(mx, p["mega.wh1.weight"], p["mega.wh1.bias"]) + F.linear(attn, p["mega.wh2.weight"])
    y1 = h + x
    # normalised FFN
    n = F.layer_norm(y1, (D,), p["nffn.norm.weight"] + 1.0, p["nffn.norm.bias"], eps)
    if swiglu:
        hid = F.silu(F.linear(n, p["nffn.fc1.weight"])) * F.linear(n, p["nffn.fc3.weight"])
    else:
        hid = F.silu(F.linear(n, p["nffn.fc1.weight"]))
    return F.linear(hid, p["nffn.fc2.weight"]) + x
