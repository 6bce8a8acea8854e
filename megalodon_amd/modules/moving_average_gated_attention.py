"""`MovingAverageGatedAttention` and `MegaBlock` for one device
(megalodon/modules/moving_average_gated_attention.py:145-353,
megalodon/model/mega.py:43-88): TimestepNorm -> CEMA -> RMSNorm -> z/q/k, v, r
projections -> chunk attention -> gate -> wh1 + wh2 -> residual, then the
normalised feed-forward network.  World size 1: the Column/RowParallelLinear
layers are `nn.Linear`, the chunk-parallel send/recv branches are not part of
this path.  The three dropouts sit where the reference has them (:316, :336,
:340; DropKey inside the attention operator).  With `cache` = (attention cache, (count, mean, var)
of TimestepNorm, EMA state) a sequence can be fed piece by piece (:283-297,
:306-308, :345-346): every piece continues the running statistics, the EMA
state and the unfinished attention chunk of the one before."""
import math
from typing import Optional

import torch
import torch.nn.functional as F
from torch import Tensor, nn
from torch.nn import Parameter

from .. import extension as megalodon_ops
from ..fused_ops import memory_efficient_dropout, qk_norm_rotary, silu_mul, transpose_last2
from .chunk_attention import _InnerAttention
from .complex_exponential_moving_average import MultiHeadComplexEMA
from .linear import Linear, linear_group
from .layer_norm import FusedRMSNorm
from .normalized_feedforward_network import NormalizedFeedForwardNetwork
from .timestep_norm import TimestepNorm


class MovingAverageGatedAttention(nn.Module):
    """Exponential Moving Average Gated Attention."""

    def __init__(self, mdim: int, zdim: int, hdim: int, ndim: int, num_heads: int, dropout: float = 0.0,
                 attention_dropout: float = 0.0, hidden_dropout: float = 0.0, chunk_size: int = 2048,
                 efficient_attn: Optional[str] = "fused", norm_num_groups: Optional[int] = None,
                 norm_affine: bool = True, norm_eps: float = 1e-5, init_std: float = 0.02):
        super().__init__()
        self.dropout = dropout
        self.attention_dropout = attention_dropout
        self.hidden_dropout = hidden_dropout
        self.mdim, self.hdim, self.zdim, self.ndim = mdim, hdim, zdim, ndim
        self.num_heads = num_heads
        assert zdim % num_heads == 0 and hdim % num_heads == 0
        self.z_head_dim = zdim // num_heads
        self.v_head_dim = hdim // num_heads
        self.local_heads = num_heads
        self.chunk_size = chunk_size
        self.efficient_attn = efficient_attn

        self.timenorm = TimestepNorm(mdim, norm_num_groups, eps=norm_eps)
        self.cema = MultiHeadComplexEMA(mdim, ndim)
        self.rmsnorm = FusedRMSNorm(mdim, elementwise_affine=norm_affine, eps=norm_eps)
        self.znorm = FusedRMSNorm(self.z_head_dim, elementwise_affine=False, eps=norm_eps)

        self.wv = Linear(mdim, hdim, bias=True)
        self.wz = Linear(mdim, zdim, bias=True)
        self.wr = Linear(mdim, hdim, bias=True)
        self.wh1 = Linear(mdim, mdim, bias=True)
        self.wh2 = Linear(hdim, mdim, bias=False)
        for lin in (self.wv, self.wz, self.wr, self.wh1, self.wh2):
            nn.init.normal_(lin.weight, mean=0.0, std=init_std)
            if lin.bias is not None:
                nn.init.zeros_(lin.bias)
        self.inner_attention = _InnerAttention(self.z_head_dim, self.v_head_dim, self.local_heads,
                                               self.chunk_size, attention_dropout, efficient_attn)
        self.gamma = Parameter(torch.zeros(2, self.z_head_dim * self.local_heads))
        self.beta = Parameter(torch.zeros(2, self.z_head_dim * self.local_heads))

    def forward(self, x: Tensor, freqs_cis: Optional[Tensor] = None, mask: Optional[Tensor] = None, cache=None):
        bsz, seq_len, _ = x.size()
        residual = x

        if cache is not None:
            cache_attn, cache_norm, hx = cache
            prev_count, prev_mean, prev_var = cache_norm
        else:
            prev_count, prev_mean, prev_var = None, None, None
            cache_attn, hx = None, None

        # B x L x D
        out_tsn, prev_count, prev_mean, prev_var = self.timenorm(x, prev_count, prev_mean, prev_var)
        # B x D x L
        out_cema, hx = self.cema(transpose_last2(out_tsn), hx, compute_last_state=cache_attn is not None)
        if cache is not None:
            cache_norm = (prev_count.detach(), prev_mean.detach(), prev_var.detach())
            hx = None if hx is None else hx.detach()
        # B x L x D
        out_cema = transpose_last2(out_cema)
        mx = self.rmsnorm(out_cema)
        mx = memory_efficient_dropout(mx, self.hidden_dropout, self.training)

        # the three projections of mx: one accumulation of its gradient in the backward
        z, r, h1 = linear_group(mx, (self.wz, self.wr, self.wh1))
        if (not self.znorm.elementwise_affine
                and megalodon_ops.qk_norm_rotary_supported(z, self.gamma, self.z_head_dim)
                and (freqs_cis is None or freqs_cis.shape[0] == min(seq_len, self.chunk_size))):
            # per-head norm, both affine maps and the rotary product in one pass over z:
            # position = index inside the chunk, which is what _InnerAttention applies
            # before (short piece) or after (long sequence) its chunk split
            q, k = qk_norm_rotary(z, self.gamma, self.beta, freqs_cis, self.z_head_dim, self.znorm.eps)
            freqs_cis = None
        else:
            # B x L x S -> B x L x H x S/H -> B x L x S
            z = self.znorm(z.view(bsz, seq_len, self.local_heads, self.z_head_dim)).view(bsz, seq_len, -1)
            # B x L x 1 x S -> B x L x 2 x S
            gamma = (self.gamma + 1.0) / math.sqrt(self.z_head_dim)
            z = z.unsqueeze(2) * gamma + self.beta
            q, k = torch.unbind(z, dim=2)

        # B x L x E
        v = F.silu(self.wv(out_tsn))

        attn, cache_attn = self.inner_attention(q.contiguous(), k.contiguous(), v, mask, freqs_cis, cache_attn)
        # attn * silu(r) in one pass
        attn = memory_efficient_dropout(silu_mul(r, attn), self.hidden_dropout, self.training)

        # B x L x E -> B x L x D
        h = self.wh2(attn, residual=h1)   # wh1(mx) + wh2(attn), the sum formed inside the GEMM
        h = memory_efficient_dropout(h, self.dropout, self.training)
        out = h + residual
        if cache is not None:
            cache = (cache_attn, cache_norm, hx)
        return out, cache

    def extra_repr(self) -> str:
        return 'edim={}, zdim={}, hdim={}, heads={}, chunk={}, eff_attn={}'.format(
            self.mdim, self.zdim, self.hdim, self.num_heads, self.chunk_size, self.efficient_attn)


class MegaBlock(nn.Module):
    """One Megalodon layer: gated attention + normalised FFN (model/mega.py:43-88)."""

    def __init__(self, model_dim: int, z_dim: int, value_dim: int, num_heads: int, cema_ndim: int,
                 chunk_size: int, ffn_hidden_dim: int, norm_num_groups: int, swiglu: bool = True,
                 efficient_attn: Optional[str] = "fused", norm_affine: bool = True, norm_eps: float = 1e-5,
                 rescale_nffn: bool = False, layer_id: int = 0, init_std: float = 0.02, dropout: float = 0.0,
                 attention_dropout: float = 0.0, hidden_dropout: float = 0.0):
        super().__init__()
        self.layer_id = layer_id
        self.mega = MovingAverageGatedAttention(
            mdim=model_dim, zdim=z_dim, hdim=value_dim, num_heads=num_heads, ndim=cema_ndim,
            dropout=dropout, attention_dropout=attention_dropout, hidden_dropout=hidden_dropout,
            chunk_size=chunk_size, efficient_attn=efficient_attn, norm_num_groups=norm_num_groups,
            norm_affine=norm_affine, norm_eps=norm_eps, init_std=init_std)
        rescale = 0.1 * (0.5 ** layer_id) if rescale_nffn else None
        self.nffn = NormalizedFeedForwardNetwork(
            model_dim=model_dim, ffn_hidden_dim=ffn_hidden_dim, dropout=dropout, hidden_dropout=hidden_dropout,
            swiglu=swiglu, norm_affine=norm_affine,
            norm_eps=norm_eps, rescale=rescale, init_std=init_std)

    def forward(self, x: Tensor, freqs_cis: Optional[Tensor] = None, mask: Optional[Tensor] = None, cache=None):
        y, cache = self.mega(x, freqs_cis, mask, cache)
        out = self.nffn(y, x)
        return out, cache
