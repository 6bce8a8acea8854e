"""`_InnerAttention` with the reference's constructor and forward
(megalodon/modules/moving_average_gated_attention.py:43-142): view the
sequence as chunks, rotary on q/k, causal attention inside each chunk through
the fused operator.  The rotary product is plain PyTorch (restating
megalodon/modules/rotary_positional_embedding.py:53-77).  With a key/value
cache (:92-101) the cached keys and values of the unfinished chunk are put in
front of the new ones: the fused operator then sees L2 > L1 (row r attends to
keys 0 .. L2 - L1 + r), and a single new token attends to everything (:132-135)."""
from typing import Optional, Tuple

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from ..fused_ops import memory_efficient_dropout, swift_efficient_attention


def apply_rotary_emb(xq: Tensor, xk: Tensor, freqs_cis: Optional[Tensor], backward: bool = False):
    if freqs_cis is None:
        return xq, xk
    if backward:
        freqs_cis = freqs_cis.conj()
    xq_ = torch.view_as_complex(xq.float().reshape(*xq.shape[:-1], -1, 2))
    xk_ = torch.view_as_complex(xk.float().reshape(*xk.shape[:-1], -1, 2))
    freqs_cis = freqs_cis.unsqueeze(1)  # C x 1 x D/2
    xq_out = torch.view_as_real(xq_ * freqs_cis).flatten(3)
    xk_out = torch.view_as_real(xk_ * freqs_cis).flatten(3)
    return xq_out.type_as(xq), xk_out.type_as(xk)


def get_efficient_attention_function(attn_name: str):
    return {"swift": swift_efficient_attention, "fused": swift_efficient_attention}[attn_name]


class _InnerAttention(nn.Module):
    """Inner attention"""

    def __init__(self, z_head_dim: int, v_head_dim: int, n_heads: int, chunk_size: int, dropout: float,
                 efficient_attn: Optional[str]):
        super().__init__()
        self.z_head_dim = z_head_dim
        self.v_head_dim = v_head_dim
        self.n_heads = n_heads
        self.chunk_size = chunk_size
        self.dropout = dropout
        self.efficient_attn = efficient_attn
        self.attn_fn = get_efficient_attention_function(efficient_attn) if efficient_attn is not None else None

    def forward(self, xq: Tensor, xk: Tensor, xv: Tensor, mask: Optional[Tensor], freqs_cis: Optional[Tensor],
                cache: Optional[Tuple[Tensor, Tensor, int]] = None):
        bs, slen, _ = xq.shape
        xq = xq.view(bs, slen, self.n_heads, self.z_head_dim)
        xk = xk.view(bs, slen, self.n_heads, self.z_head_dim)
        xv = xv.view(bs, slen, self.n_heads, self.v_head_dim)

        # shorter than a chunk: rope before the cached keys are put in front
        if slen <= self.chunk_size:
            xq, xk = apply_rotary_emb(xq, xk, freqs_cis=freqs_cis, backward=False)

        new_cache = None
        clen = slen
        if cache is not None:
            cache_k, cache_v, count = cache
            xk = torch.cat([cache_k, xk], dim=1)
            xv = torch.cat([cache_v, xv], dim=1)
            clen = count + slen
            # what is left of the last, unfinished chunk goes to the next call
            new_count = clen % self.chunk_size
            new_cache = (xk.detach()[:, clen - new_count:], xv.detach()[:, clen - new_count:], new_count)

        if self.chunk_size < slen:
            nc = slen // self.chunk_size
            xq = xq.reshape(bs * nc, self.chunk_size, self.n_heads, self.z_head_dim)
        if self.chunk_size < clen:
            nc = clen // self.chunk_size
            xk = xk.reshape(bs * nc, self.chunk_size, self.n_heads, self.z_head_dim)
            xv = xv.reshape(bs * nc, self.chunk_size, self.n_heads, self.v_head_dim)
        # seq length > chunk: rope after the chunk split
        if slen > self.chunk_size:
            xq, xk = apply_rotary_emb(xq, xk, freqs_cis=freqs_cis, backward=False)

        if self.efficient_attn is None:
            # unfused branch of the reference (:116-129), kept for comparison
            xq, xk, xv = xq.transpose(1, 2), xk.transpose(1, 2), xv.transpose(1, 2)
            assert mask is not None
            scores = torch.matmul(xq, xk.transpose(2, 3)) + mask
            scores = F.softmax(scores, dim=-1, dtype=torch.float32).to(xq)
            scores = memory_efficient_dropout(scores, self.dropout, self.training)
            output = torch.matmul(scores, xv).transpose(1, 2).contiguous()
        else:
            assert mask is None
            use_causal_mask = not (slen == 1 and cache is not None)
            output = self.attn_fn(xq.contiguous(), xk.contiguous(), xv.contiguous(), 1.0, self.dropout,
                                  use_causal_mask, self.training)

        output = output.reshape(bs, slen, -1)
        return output, new_cache

    def extra_repr(self) -> str:
        return 'heads={}, z_head_dim={}, v_head_dim={}, chunk={}'.format(
            self.n_heads, self.z_head_dim, self.v_head_dim, self.chunk_size)
