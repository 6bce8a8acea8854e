"""Pins the attention oracle: textbook properties and the agreement of the
reference's explicit backward formulas with autograd."""
import torch

from oracle import attention as oa


def _qkv(B, L, N, H1, H2, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, L, N, H1, generator=g, dtype=torch.float64) / H1 ** 0.5
    k = torch.randn(B, L, N, H1, generator=g, dtype=torch.float64) / H1 ** 0.5
    v = torch.randn(B, L, N, H2, generator=g, dtype=torch.float64)
    dy = torch.randn(B, L, N, H2, generator=g, dtype=torch.float64)
    return q, k, v, dy


def test_row0_sees_only_first_key_and_rows_sum_to_one():
    q, k, v, _ = _qkv(2, 9, 3, 4, 5, 0)
    y, p = oa.chunk_attention_fwd(q, k, v, 1.0, True)
    assert torch.allclose(y[:, 0], v[:, 0], atol=1e-14)
    assert torch.allclose(p.sum(-1), torch.ones_like(p.sum(-1)), atol=1e-14)
    assert p.triu(1).abs().max() == 0


def test_bruteforce_loops():
    q, k, v, _ = _qkv(1, 6, 2, 3, 4, 1)
    y, _ = oa.chunk_attention_fwd(q, k, v, 0.7, True)
    for n in range(2):
        for r in range(6):
            s = torch.tensor([0.7 * (q[0, r, n] * k[0, c, n]).sum() for c in range(r + 1)], dtype=torch.float64)
            w = torch.exp(s - s.max())
            w = w / w.sum()
            want = sum(w[c] * v[0, c, n] for c in range(r + 1))
            assert torch.allclose(y[0, r, n], want, atol=1e-13)


def test_chunks_are_independent_and_permute():
    q, k, v, _ = _qkv(4, 7, 2, 4, 3, 2)
    y, _ = oa.chunk_attention_fwd(q, k, v)
    perm = torch.tensor([2, 0, 3, 1])
    yp, _ = oa.chunk_attention_fwd(q[perm], k[perm], v[perm])
    assert torch.allclose(yp, y[perm], atol=1e-14)


def test_bottom_right_alignment_with_longer_keys():
    q, k, v, _ = _qkv(1, 8, 1, 4, 3, 3)
    y_full, _ = oa.chunk_attention_fwd(q, k, v)
    y_tail, _ = oa.chunk_attention_fwd(q[:, 5:], k, v)
    assert torch.allclose(y_tail, y_full[:, 5:], atol=1e-14)


def test_explicit_backward_formulas_equal_autograd():
    for causal in (True, False):
        q, k, v, dy = _qkv(2, 10, 2, 4, 6, 4)
        a = oa.chunk_attention_bwd(dy, q, k, v, 0.9, causal)
        b = oa.chunk_attention_bwd_formulas(dy, q, k, v, 0.9, causal)
        for x, y_ in zip(a, b):
            assert torch.allclose(x, y_, atol=1e-12)
