"""Rotary position factors (mirror of
megalodon/modules/rotary_positional_embedding.py:8-50): `freqs_cis[t, j] =
exp(i t base^(-2j / dim))` for positions inside a chunk.  The product itself is
`apply_rotary_emb` in chunk_attention.py, or part of the fused z -> (q, k)
kernel when the block runs on the GPU."""
import warnings
from typing import Optional

import torch
from torch import nn

from .chunk_attention import apply_rotary_emb


class RotaryEmbedding(nn.Module):
    def __init__(self, embed_dim: int, max_positions: int, base: Optional[float] = None):
        super().__init__()
        assert embed_dim % 2 == 0
        self.embed_dim = embed_dim
        self.max_positions = max_positions
        self.base = 10000 if base is None else base
        exponents = torch.arange(0, embed_dim, 2, dtype=torch.float32) / embed_dim
        self.register_buffer("freqs", 1.0 / torch.tensor(float(self.base)) ** exponents)
        self.freqs_cis: Optional[torch.Tensor] = None

    @torch.no_grad()
    def _table(self, positions: int) -> torch.Tensor:
        """exp(i t f_j) for t < positions: complex64, (positions, dim / 2)."""
        t = torch.arange(positions, dtype=torch.float32, device=self.freqs.device)
        angles = torch.outer(t, self.freqs.float())
        return torch.polar(torch.ones_like(angles), angles)

    def get_freqs_cis(self, start: int, end: int) -> torch.Tensor:
        """Rows start .. end-1 of the table; the table grows (with a warning, as
        in the reference :36-42) when `end` lies beyond it."""
        have = 0 if self.freqs_cis is None else self.freqs_cis.shape[0]
        if end > have:
            if end > self.max_positions:
                warnings.warn(f"Extending rotary range from {self.max_positions} to {end}")
                self.max_positions = end
            self.freqs_cis = self._table(self.max_positions)
        return self.freqs_cis[start:end]

    def forward(self, xq, xk, start: int):
        freqs_cis = self.get_freqs_cis(start, start + xq.shape[1])
        return apply_rotary_emb(xq, xk, freqs_cis=freqs_cis, backward=False)

    def extra_repr(self) -> str:
        return f"dim={self.embed_dim}, max positions={self.max_positions}, base={self.base:.1f}"
