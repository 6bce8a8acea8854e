"""`_InnerAttention` with the reference's constructor and forward
(megalodon/modules/moving_average_gated_attention.py:43-142): view the
sequence as chunks, rotary on q/k, causal attention inside each chunk through
the fused operator.  The rotary product is plain PyTorch (restating
megalodon/modules/rotary_positional_embedding.py:53-77); the key/value cache
branch (:92-101) belongs to cached inference and is not implemented."""
from typing import Optional, Tuple

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from ..fused_ops import swift_efficient_attention


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
        if cache is not None:
            raise NotImplementedError("key/value cache (cached inference) is not implemented")
        bs, slen, _ = xq.shape
        xq = xq.view(bs, slen, self.n_heads, self.z_head_dim)
        xk = xk.view(bs, slen, self.n_heads, self.z_head_dim)
        xv = xv.view(bs, slen, self.n_heads, self.v_head_dim)

        # shorter than a chunk: rope before chunking
        if slen <= self.chunk_size:
            xq, xk = apply_rotary_emb(xq, xk, freqs_cis=freqs_cis, backward=False)

        if self.chunk_size < slen:
            nc = slen // self.chunk_size
            xq = xq.reshape(bs * nc, self.chunk_size, self.n_heads, self.z_head_dim)
            xk = xk.reshape(bs * nc, self.chunk_size, self.n_heads, self.z_head_dim)
            xv = xv.reshape(bs * nc, self.chunk_size, self.n_heads, self.v_head_dim)
            # seq length > chunk: rope after the chunk split
            xq, xk = apply_rotary_emb(xq, xk, freqs_cis=freqs_cis, backward=False)

        if self.efficient_attn is None:
            # unfused branch of the reference (:116-129), kept for comparison
            xq, xk, xv = xq.transpose(1, 2), xk.transpose(1, 2), xv.transpose(1, 2)
            assert mask is not None
            scores = torch.matmul(xq, xk.transpose(2, 3)) + mask
            scores = F.softmax(scores, dim=-1, dtype=torch.float32).to(xq)
            output = torch.matmul(scores, xv).transpose(1, 2).contiguous()
        else:
            assert mask is None
            output = self.attn_fn(xq, xk, xv, 1.0, self.dropout, True, self.training)

        output = output.reshape(bs, slen, -1)
        return output, None

    def extra_repr(self) -> str:
        return 'heads={}, z_head_dim={}, v_head_dim={}, chunk={}'.format(
            self.n_heads, self.z_head_dim, self.v_head_dim, self.chunk_size)
