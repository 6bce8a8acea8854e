"""`NormalizedFeedForwardNetwork` (megalodon/modules/normalized_feedforward_network.py:15-98)
for model-parallel world size 1: Column/RowParallelLinear are plain `nn.Linear`
(megalodon/modules/model_parallel/layers.py:222-235,321-341); the two dropouts
sit where the reference has them (:83-90)."""
import torch
import torch.nn.functional as F
from torch import nn

from ..fused_ops import memory_efficient_dropout, silu_mul
from .linear import Linear, linear_group
from .layer_norm import FusedLayerNorm


class NormalizedFeedForwardNetwork(nn.Module):
    def __init__(self, model_dim, ffn_hidden_dim, dropout=0.0, hidden_dropout=0.0, swiglu=False,
                 norm_affine=True, norm_eps=1e-5, rescale=None, init_std=0.02):
        super().__init__()
        self.dropout = dropout
        self.hidden_dropout = hidden_dropout
        self.model_dim = model_dim
        self.hidden_dim = ffn_hidden_dim
        self.swiglu = swiglu
        self.rescale_init = rescale
        self.norm = FusedLayerNorm(model_dim, elementwise_affine=norm_affine, eps=norm_eps)
        self.fc1 = Linear(model_dim, ffn_hidden_dim, bias=False)
        self.fc2 = Linear(ffn_hidden_dim, model_dim, bias=False)
        self.fc3 = Linear(model_dim, ffn_hidden_dim, bias=False) if swiglu else None
        for lin in (self.fc1, self.fc2, self.fc3):
            if lin is not None:
                nn.init.normal_(lin.weight, mean=0.0, std=init_std)
        if rescale is None:
            self.register_parameter('alpha', None)
        else:
            assert rescale > 0., 'Layer scale init value should be positive.'
            self.alpha = nn.Parameter(torch.full((model_dim,), rescale))

    def rescale(self, x: torch.Tensor) -> torch.Tensor:
        return x if self.alpha is None else (self.alpha * x)

    def forward(self, x, residual):
        x = self.norm(x)
        if self.swiglu:
            hidden = silu_mul(*linear_group(x, (self.fc1, self.fc3)))
        else:
            hidden = F.silu(self.fc1(x))
        hidden = memory_efficient_dropout(hidden, self.hidden_dropout, self.training)
        if self.alpha is None and (self.dropout == 0.0 or not self.training):
            return self.fc2(hidden, residual=residual)   # fc2(hidden) + residual, the sum formed inside the GEMM
        x = self.fc2(hidden)
        x = memory_efficient_dropout(x, self.dropout, self.training)
        return self.rescale(x) + residual

    def extra_repr(self) -> str:
        return 'dim={}, hdim={}, swiglu={}, rescale={}'.format(self.model_dim, self.hidden_dim, self.swiglu,
                                                             self.rescale_init)
