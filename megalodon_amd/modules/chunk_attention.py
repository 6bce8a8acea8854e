"""`_InnerAttention`: attention that is causal inside chunks of `chunk_size`
positions and blind across them, behind the reference's constructor and call
signature (megalodon/modules/moving_average_gated_attention.py:43-142).

What the call does, in this build's terms:
  1. split the projections into heads (layout B, L, heads, dim: the fused operator's own);
  2. turn the *new* queries and keys by the rotary angles of their position inside the chunk
     (`freqs_cis[t]` for chunk position t; rotary_positional_embedding.py:53-77).  Cached keys
     were turned when they were new, so this happens before the cache is joined;
  3. with a cache `(keys, values, count)`: put the unfinished chunk's keys / values in front and
     hand the new unfinished tail on to the next call (:92-101);
  4. fold whole chunks into the batch axis and run the fused operator, which takes L2 >= L1
     (row r sees keys 0 .. L2 - L1 + r) and, for one new token on a cache, every key (:132-135).
"""
from typing import Optional, Tuple

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from ..fused_ops import memory_efficient_dropout, swift_efficient_attention

_FUSED = {"swift": swift_efficient_attention, "fused": swift_efficient_attention}


def _turn(x: Tensor, freqs_cis: Tensor) -> Tensor:
    """Rotate the (even, odd) feature pairs of x (..., C, heads, dim) by the unit complex numbers
    freqs_cis (C, dim / 2), in float32, and round back to x's dtype."""
    pairs = x.float().unflatten(-1, (-1, 2))
    re, im = pairs[..., 0], pairs[..., 1]
    c, s = freqs_cis.real[:, None, :], freqs_cis.imag[:, None, :]
    return torch.stack((re * c - im * s, re * s + im * c), dim=-1).flatten(-2).to(x.dtype)


def apply_rotary_emb(xq: Tensor, xk: Tensor, freqs_cis: Optional[Tensor], backward: bool = False):
    """Rotary product on a (query, key) pair; `backward` turns the other way (the gradient's map)."""
    if freqs_cis is None:
        return xq, xk
    f = freqs_cis.conj() if backward else freqs_cis
    return _turn(xq, f), _turn(xk, f)


def get_efficient_attention_function(attn_name: str):
    return _FUSED[attn_name]


class _InnerAttention(nn.Module):
    """Chunk-causal attention over (B, L, heads * dim) projections."""

    def __init__(self, z_head_dim: int, v_head_dim: int, n_heads: int, chunk_size: int, dropout: float,
                 efficient_attn: Optional[str]):
        super().__init__()
        self.z_head_dim, self.v_head_dim = z_head_dim, v_head_dim
        self.n_heads, self.chunk_size = n_heads, chunk_size
        self.dropout = dropout
        self.efficient_attn = efficient_attn
        self.attn_fn = None if efficient_attn is None else _FUSED[efficient_attn]

    def _chunks(self, t: Tensor) -> Tensor:
        """(B, n * chunk, heads, dim) -> (B * n, chunk, heads, dim); shorter sequences pass."""
        if t.shape[1] <= self.chunk_size:
            return t
        return t.reshape(-1, self.chunk_size, *t.shape[2:])

    def forward(self, xq: Tensor, xk: Tensor, xv: Tensor, mask: Optional[Tensor], freqs_cis: Optional[Tensor],
                cache: Optional[Tuple[Tensor, Tensor, int]] = None):
        batch, new_len = xq.shape[:2]
        q = xq.unflatten(-1, (self.n_heads, self.z_head_dim))
        k = xk.unflatten(-1, (self.n_heads, self.z_head_dim))
        v = xv.unflatten(-1, (self.n_heads, self.v_head_dim))

        if freqs_cis is not None:
            # chunk position of a new token = its row in the chunk view
            shape_q, shape_k = q.shape, k.shape
            q, k = apply_rotary_emb(self._chunks(q), self._chunks(k), freqs_cis)
            q, k = q.reshape(shape_q), k.reshape(shape_k)

        carried = None
        if cache is not None:
            old_k, old_v, old_len = cache
            k, v = torch.cat((old_k, k), dim=1), torch.cat((old_v, v), dim=1)
            total = old_len + new_len
            tail = total % self.chunk_size  # steps of the chunk still open after this call
            carried = (k.detach()[:, total - tail:], v.detach()[:, total - tail:], tail)

        q, k, v = self._chunks(q), self._chunks(k), self._chunks(v)
        if self.attn_fn is not None:
            assert mask is None
            one_token_on_cache = new_len == 1 and cache is not None
            out = self.attn_fn(q.contiguous(), k.contiguous(), v.contiguous(), 1.0, self.dropout,
                               not one_token_on_cache, self.training)
        else:
            # the reference's unfused branch (:116-129): additive mask, float32 softmax
            assert mask is not None
            qh, kh, vh = (t.transpose(1, 2) for t in (q, k, v))
            prob = F.softmax(qh @ kh.transpose(2, 3) + mask, dim=-1, dtype=torch.float32).to(qh.dtype)
            prob = memory_efficient_dropout(prob, self.dropout, self.training)
            out = (prob @ vh).transpose(1, 2).contiguous()
        return out.reshape(batch, new_len, -1), carried

    def extra_repr(self) -> str:
        return (f"heads={self.n_heads}, z_head_dim={self.z_head_dim}, v_head_dim={self.v_head_dim}, "
                f"chunk={self.chunk_size}")
