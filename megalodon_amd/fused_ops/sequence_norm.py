"""`sequence_norm(x, gamma, beta, padding_mask=None, num_groups=None, eps=1e-5,
length_last=False) -> y`: every (sequence, feature group) normalised over its
unmasked steps and the group's features, differentiable in x, gamma and beta.
The reference ships these operators without a Python wrapper
(megalodon/csrc/ops/sequence_norm.cc:1066-1071); this one follows the pattern
of its other fused ops.  `num_groups=None` is one group per feature."""
from .. import extension as ops
from ._autograd import fused_op


def _run(x, gamma, beta, padding_mask=None, num_groups=None, eps=1e-5, length_last=False):
    features = x.size(1) if length_last else x.size(-1)
    groups = features if num_groups is None else num_groups
    y, count, mean, rstd = ops.group_sequence_norm_fwd(x, gamma, beta, padding_mask, groups, eps, length_last)
    return y, (x, count, mean, rstd, gamma, padding_mask), (groups, length_last)


def _grad(consts, saved, y_grad):
    x, count, mean, rstd, gamma, padding_mask = saved
    dx, dgamma, dbeta = ops.group_sequence_norm_bwd(y_grad, x, count, mean, rstd, gamma, padding_mask, *consts)
    return dx, dgamma, dbeta, None, None, None, None


SequenceNormFunc = fused_op("SequenceNormFunc", _run, _grad, doc=__doc__)
sequence_norm = SequenceNormFunc.apply
