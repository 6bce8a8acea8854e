"""`TimestepNorm` / `TimestepNormFunc` with the reference's signatures
(megalodon/modules/timestep_norm.py:13-131), minus the model-parallel split
(world size 1: features_per_partition = num_features).  The module always
routes through the group operator, as the reference does (:123-125); the
non-group call form (``num_groups=None`` in the function) maps to one group
per feature, which is the same arithmetic."""
from typing import Optional, Tuple

import torch
import torch.nn as nn
from torch.nn.parameter import Parameter

from .. import extension as ops
from ..fused_ops._autograd import fused_op


def _run(x, prev_count, prev_mean, prev_var, gamma, beta, padding_mask=None, num_groups=None, eps=1e-5):
    groups = x.size(-1) if num_groups is None else num_groups
    # cummean / cumrstd go to the backward and nowhere else, so they are kept time-last, (B, G, L):
    # the kernels then write and read them as whole lines
    time_last = x.dtype != torch.float64
    y, count, mean, var, cummean, cumrstd = ops.group_timestep_norm_fwd(
        x, prev_count, prev_mean, prev_var, gamma, beta, padding_mask, groups, eps, stats_time_last=time_last)
    return (y, count, mean, var), (x, prev_mean, count, cummean, cumrstd, gamma, padding_mask), (groups, time_last)


def _grad(consts, saved, y_grad, _count_grad, mean_grad, var_grad):
    groups, time_last = consts
    x, prev_mean, count, cummean, cumrstd, gamma, padding_mask = saved
    # an output nobody used arrives as None
    mean_grad = torch.zeros_like(prev_mean) if mean_grad is None else mean_grad
    var_grad = torch.zeros_like(prev_mean) if var_grad is None else var_grad
    dx, dprev_mean, dprev_var, dgamma, dbeta = ops.group_timestep_norm_bwd(
        y_grad, mean_grad, var_grad, x, prev_mean, count, cummean, cumrstd, gamma, padding_mask, groups,
        stats_time_last=time_last)
    #      x   count  prev_mean   prev_var   gamma   beta   mask  groups eps
    return dx, None, dprev_mean, dprev_var, dgamma, dbeta, None, None, None


TimestepNormFunc = fused_op(
    "TimestepNormFunc", _run, _grad, non_differentiable=(1,),
    doc="(y, count, mean, var) = timestep_norm(x, prev_count, prev_mean, prev_var, gamma, beta, "
        "padding_mask=None, num_groups=None, eps=1e-5); count is not differentiable.")
timestep_norm = TimestepNormFunc.apply


class TimestepNorm(nn.Module):
    """Cumulative group normalisation over time.  State dict as the reference's
    (`prior_count` buffer; `prior_mean`, `prior_logv` parameters when
    `prior_count > 0`, buffers otherwise; `weight` stored as gamma - 1; `bias`).
    One group per feature (`num_groups=None`) needs a prior of more than one
    step, as in the reference (:79-83)."""

    def __init__(self, num_features: int, num_groups: Optional[int] = None, prior_count: int = 0,
                 eps: float = 1e-5) -> None:
        super().__init__()
        per_feature = num_groups is None or num_groups == num_features
        groups = num_features if per_feature else num_groups
        if per_feature:
            assert prior_count > 1
        else:
            assert num_features % groups == 0
        self.num_features, self.num_groups, self.eps = num_features, num_groups, eps
        self._prior_count = prior_count
        # world size 1: a partition is the whole feature axis
        self.features_per_partition, self.groups_per_partition = num_features, groups

        self.register_buffer("prior_count", torch.tensor(prior_count, dtype=torch.int64))
        for stat in ("prior_mean", "prior_logv"):
            if prior_count > 0:
                self.register_parameter(stat, Parameter(torch.zeros(groups)))
            else:
                self.register_buffer(stat, torch.zeros(groups))
        for affine in ("weight", "bias"):
            self.register_parameter(affine, Parameter(torch.zeros(num_features)))

    def forward(
        self,
        x: torch.Tensor,
        prev_count: Optional[torch.Tensor] = None,
        prev_mean: Optional[torch.Tensor] = None,
        prev_var: Optional[torch.Tensor] = None,
        padding_mask: Optional[torch.Tensor] = None,
    ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
        B = x.size(0)
        # a missing state is the learned prior, one copy per sequence (:116-121)
        count = self.prior_count.expand(B).contiguous() if prev_count is None else prev_count
        mean = self.prior_mean.expand(B, -1).contiguous() if prev_mean is None else prev_mean
        var = self.prior_logv.exp().expand(B, -1).contiguous() if prev_var is None else prev_var
        # the operator takes statistics and affine parameters in x's dtype
        # (timestep_norm_kernel.cu:1270-1273 reads them as data_ptr<T>())
        return timestep_norm(x, count, mean.to(x), var.to(x), (self.weight + 1.0).to(x), self.bias.to(x),
                             padding_mask, self.groups_per_partition, self.eps)

    def extra_repr(self) -> str:
        return (f"num_features={self.num_features} ({self.features_per_partition}), "
                f"num_groups={self.num_groups} ({self.groups_per_partition}), "
                f"prior_count={self._prior_count}, eps={self.eps}")
