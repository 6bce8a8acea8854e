"""`FusedLayerNorm` / `FusedRMSNorm` with the reference's parameterisation
(megalodon/modules/layer_norm.py:14-66: stored weight is `gamma - 1`; the
reference adds 1 and calls apex's fused_layer_norm_cuda).  On the GPU the
normalisation over the last axis runs as one streaming kernel that takes the
stored weight as it is; CPU tensors and multi-axis shapes use PyTorch's
layer_norm / rms_norm."""
import numbers

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..fused_ops import layer_norm_plus_one


def _param_dtype(weight, input_):
    return input_.dtype if weight is None else weight.dtype


class FusedLayerNorm(nn.Module):
    def __init__(self, normalized_shape, eps=1e-5, elementwise_affine=True):
        super().__init__()
        if isinstance(normalized_shape, numbers.Integral):
            normalized_shape = (normalized_shape,)
        self.normalized_shape = torch.Size(normalized_shape)
        self.eps = eps
        self.elementwise_affine = elementwise_affine
        if self.elementwise_affine:
            self.weight = nn.Parameter(torch.zeros(*normalized_shape))
            self.bias = nn.Parameter(torch.zeros(*normalized_shape))
        else:
            self.register_parameter("weight", None)
            self.register_parameter("bias", None)

    def forward(self, input_):
        if input_.is_cuda and len(self.normalized_shape) == 1 and input_.dtype == _param_dtype(self.weight, input_):
            return layer_norm_plus_one(input_, self.weight, self.bias, self.eps, False)
        weight = None if self.weight is None else self.weight + 1.0
        return F.layer_norm(input_, self.normalized_shape, weight, self.bias, self.eps)

    def extra_repr(self):
        return "{normalized_shape}, eps={eps}, elementwise_affine={elementwise_affine}".format(**self.__dict__)


class FusedRMSNorm(nn.Module):
    def __init__(self, normalized_shape, eps=1e-5, elementwise_affine=True):
        super().__init__()
        if isinstance(normalized_shape, numbers.Integral):
            normalized_shape = (normalized_shape,)
        self.normalized_shape = torch.Size(normalized_shape)
        self.eps = eps
        self.elementwise_affine = elementwise_affine
        if self.elementwise_affine:
            self.weight = nn.Parameter(torch.zeros(*normalized_shape))
        else:
            self.register_parameter("weight", None)

    def forward(self, input_):
        if input_.is_cuda and len(self.normalized_shape) == 1 and input_.dtype == _param_dtype(self.weight, input_):
            return layer_norm_plus_one(input_, self.weight, None, self.eps, True)
        weight = None if self.weight is None else self.weight + 1.0
        return F.rms_norm(input_, self.normalized_shape, weight, self.eps)

    def extra_repr(self):
        return "{normalized_shape}, eps={eps}, elementwise_affine={elementwise_affine}".format(**self.__dict__)
