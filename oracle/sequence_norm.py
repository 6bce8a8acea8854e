"""Float64 restatement of the whole-sequence (group) normalisation
(TEST INFRASTRUCTURE ONLY).

Follows megalodon/csrc/ops/sequence_norm.cc: forward :531-599 (features last)
and :601-655 (length last), backward :657-842; the per-feature operator
(:258-529) is the case num_groups = H.  Statistics are taken over the unmasked
steps and the D = H / num_groups features of a group, with the biased variance
(utils.h:144-164).
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch


def _to_blh(t: torch.Tensor, length_last: bool) -> torch.Tensor:
    return t.transpose(1, 2) if length_last else t


def group_sequence_norm_fwd(x: torch.Tensor, gamma: torch.Tensor, beta: torch.Tensor,
                            padding_mask: Optional[torch.Tensor], num_groups: int, eps: float,
                            length_last: bool = False
                            ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """(y, count, mean, rstd); y in x's layout, float64."""
    xb = _to_blh(x.double(), length_last)
    B, L, H = xb.shape
    G, D = num_groups, H // num_groups
    keep = torch.ones(B, L, dtype=torch.float64) if padding_mask is None else (~padding_mask).double()
    count = keep.sum(1).to(torch.int64)
    xg = xb.reshape(B, L, G, D)
    n = (count.double() * D).clamp(min=1).view(B, 1)
    mean = (xg * keep.view(B, L, 1, 1)).sum((1, 3)) / n
    cen = (xg - mean.view(B, 1, G, 1)) * keep.view(B, L, 1, 1)
    var = (cen * cen).sum((1, 3)) / n
    rstd = 1.0 / torch.sqrt(var + eps)
    y = (xg - mean.view(B, 1, G, 1)) * rstd.view(B, 1, G, 1)
    y = y.reshape(B, L, H) * gamma.double() + beta.double()
    y = y * keep.view(B, L, 1)
    return _to_blh(y, length_last).contiguous(), count, mean, rstd


def group_sequence_norm_bwd(dy: torch.Tensor, x: torch.Tensor, count: torch.Tensor, mean: torch.Tensor,
                            rstd: torch.Tensor, gamma: torch.Tensor, padding_mask: Optional[torch.Tensor],
                            num_groups: int, length_last: bool = False
                            ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dx, dgamma, dbeta), float64.  ds = sum dy x and db = sum dy over the
    unmasked steps of a feature; per group dsw = sum gamma ds, dbw = sum gamma db
    (sequence_norm.cc:703-710); then
    dx = rstd gamma dy + 2 c (x - mean) dv + c du with c = 1 / (count D),
    dv = rstd^3 (mean dbw - dsw) / 2, du = -rstd dbw (:717-727);
    dgamma = sum_b rstd (ds - mean db), dbeta = sum_b db (:733-748)."""
    xb = _to_blh(x.double(), length_last)
    gb = _to_blh(dy.double(), length_last)
    B, L, H = xb.shape
    G, D = num_groups, H // num_groups
    keep = torch.ones(B, L, dtype=torch.float64) if padding_mask is None else (~padding_mask).double()
    gb = gb * keep.view(B, L, 1)
    w = gamma.double()
    ds = (gb * xb).sum(1)  # (B, H)
    db = gb.sum(1)
    dsw = (ds * w).view(B, G, D).sum(2)
    dbw = (db * w).view(B, G, D).sum(2)
    u, r = mean.double(), rstd.double()
    c = 1.0 / (count.double() * D).clamp(min=1).view(B, 1)
    dv = 0.5 * r ** 3 * (u * dbw - dsw)
    du = -r * dbw
    xg = xb.view(B, L, G, D)
    dx = (r.view(B, 1, G, 1) * (gb * w).view(B, L, G, D)
          + 2.0 * (c * dv).view(B, 1, G, 1) * (xg - u.view(B, 1, G, 1)) + (c * du).view(B, 1, G, 1))
    dx = dx.reshape(B, L, H) * keep.view(B, L, 1)
    ue, re = u.repeat_interleave(D, 1), r.repeat_interleave(D, 1)
    dgamma = (re * (ds - ue * db)).sum(0)
    dbeta = db.sum(0)
    return _to_blh(dx, length_last).contiguous(), dgamma, dbeta
