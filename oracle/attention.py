"""Oracle for chunk-causal attention (float64).

Follows the reference's own unfused branch,
megalodon/modules/moving_average_gated_attention.py:116-129
(matmul + additive causal mask + float32 softmax + matmul), which is the
textbook formula; gradients by autograd.  Layout BLNH like the fused operator
(megalodon/csrc/ops/attention_kernel.cu:46-51).
"""
from __future__ import annotations

import torch


def chunk_attention_fwd(q, k, v, scale=1.0, causal=True, drop=None):
    """q (B, L1, N, H1), k (B, L2, N, H1), v (B, L2, N, H2) -> (y (B, L1, N, H2), p (B, N, L1, L2)).
    Row r sees columns 0..L2-L1+r (bottom-right aligned, softmax.cuh:99-100).
    `drop` (B, N, L1, L2) bool: DropKey (softmax.cuh:165-172) -- those scores
    become -inf before the softmax, nothing is rescaled, and a row left with
    no key is 0 (softmax.cuh:178-181)."""
    q = q.double().transpose(1, 2)
    k = k.double().transpose(1, 2)
    v = v.double().transpose(1, 2)
    L1, L2 = q.shape[2], k.shape[2]
    scores = torch.matmul(q, k.transpose(2, 3)) * scale
    if causal:
        r = torch.arange(L1).view(L1, 1)
        c = torch.arange(L2).view(1, L2)
        scores = scores.masked_fill(c > r + (L2 - L1), float("-inf"))
    if drop is not None:
        scores = scores.masked_fill(drop, float("-inf"))
        empty = torch.isinf(scores).all(dim=-1, keepdim=True)
        scores = scores.masked_fill(empty, 0.0)
        p = torch.softmax(scores, dim=-1).masked_fill(empty, 0.0)
    else:
        p = torch.softmax(scores, dim=-1)
    y = torch.matmul(p, v).transpose(1, 2).contiguous()
    return y, p


def chunk_attention_bwd(dy, q, k, v, scale=1.0, causal=True, drop=None):
    """(dq, dk, dv) by autograd over chunk_attention_fwd."""
    q = q.double().requires_grad_(True)
    k = k.double().requires_grad_(True)
    v = v.double().requires_grad_(True)
    y, _ = chunk_attention_fwd(q, k, v, scale, causal, drop)
    y.backward(dy.double())
    return q.grad, k.grad, v.grad


def chunk_attention_bwd_formulas(dy, q, k, v, scale=1.0, causal=True):
    """The reference's explicit backward (attention_kernel.cu:135-257,
    softmax.cuh:198-234): dV = P^T dY, dP = dY V^T, dS = P o (dP - rowsum(P o dP)),
    dK = scale dS^T Q, dQ = scale dS K."""
    _, p = chunk_attention_fwd(q, k, v, scale, causal)
    qh = q.double().transpose(1, 2)
    kh = k.double().transpose(1, 2)
    vh = v.double().transpose(1, 2)
    dyh = dy.double().transpose(1, 2)
    dv = torch.matmul(p.transpose(2, 3), dyh)
    dp = torch.matmul(dyh, vh.transpose(2, 3))
    ds = p * (dp - (p * dp).sum(-1, keepdim=True))
    dk = scale * torch.matmul(ds.transpose(2, 3), qh)
    dq = scale * torch.matmul(ds, kh)
    return dq.transpose(1, 2).contiguous(), dk.transpose(1, 2).contiguous(), dv.transpose(1, 2).contiguous()
