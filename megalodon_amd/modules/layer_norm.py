"""`FusedLayerNorm` / `FusedRMSNorm`: normalisation over the trailing axes with
the reference's parameterisation (megalodon/modules/layer_norm.py:14-66): the
stored `weight` is `gamma - 1` and starts at zero, so the state dict matches.
On the GPU a normalisation over the last axis is one streaming kernel that
reads the stored weight as it is (no `weight + 1` tensor is formed); CPU
tensors and multi-axis shapes go through PyTorch's layer_norm / rms_norm."""
from typing import Sequence, Union

import torch
import torch.nn.functional as F
from torch import nn

from ..fused_ops import layer_norm_plus_one


class _PlusOneNorm(nn.Module):
    """State and dispatch shared by the two norms.  `rms` drops the mean and the bias."""

    rms = False

    def __init__(self, normalized_shape: Union[int, Sequence[int]], eps: float = 1e-5,
                 elementwise_affine: bool = True):
        super().__init__()
        shape = (int(normalized_shape),) if isinstance(normalized_shape, int) else tuple(normalized_shape)
        self.normalized_shape = torch.Size(shape)
        self.eps = eps
        self.elementwise_affine = elementwise_affine
        names = ("weight",) if self.rms else ("weight", "bias")
        for name in names:
            if elementwise_affine:
                setattr(self, name, nn.Parameter(torch.zeros(shape)))
            else:
                self.register_parameter(name, None)

    def _fused(self, x: torch.Tensor) -> bool:
        same = self.weight is None or self.weight.dtype == x.dtype
        return x.is_cuda and len(self.normalized_shape) == 1 and same

    def forward(self, input_: torch.Tensor) -> torch.Tensor:
        bias = None if self.rms else self.bias
        if self._fused(input_):
            return layer_norm_plus_one(input_, self.weight, bias, self.eps, self.rms)
        gamma = self.weight + 1.0 if self.weight is not None else None
        if self.rms:
            return F.rms_norm(input_, self.normalized_shape, gamma, self.eps)
        return F.layer_norm(input_, self.normalized_shape, gamma, bias, self.eps)

    def extra_repr(self) -> str:
        return f"{tuple(self.normalized_shape)}, eps={self.eps}, elementwise_affine={self.elementwise_affine}"


class FusedLayerNorm(_PlusOneNorm):
    rms = False


class FusedRMSNorm(_PlusOneNorm):
    rms = True
