"""RMS norm on the residual stream."""
from __future__ import annotations

import torch

from .base import Norm, WeightSpec, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    """y = v * rsqrt(mean(v^2) + eps) * w over rows of ``size`` elements, where
    v is the residual stream plus the term still pending; sum, mean, rsqrt and
    products in float32.  Reference: src/kernel/cuda/norm.cu:31-48 (the weight
    product fused as in src/core/runtime/GraphOptimizer.cpp:197-229)."""

    graph_safe = True

    def __init__(self, size: int, eps: float):
        self.size = int(size)
        self.eps = float(eps)
        self.weight = None

    def weight_specs(self):
        return {"weight": WeightSpec((self.size,), "norm")}

    def load_weights(self, weights, dtype, device):
        # norm weights stay in float32 whatever the activation type is
        self.weight = weights["weight"].to(torch.float32).contiguous().to(device)

    #: ``forward`` takes ``for_linear``: its result may then be rows that lack the norm's factor,
    #: which only ``ops.linear`` understands
    for_linear_aware = True

    def forward(self, ctx, resid, delta, rows=None, for_linear=False):
        return ctx.ops.add_rmsnorm(resid, delta, self.weight, self.eps, ctx.act_dtype, rows=rows,
                                   for_linear=for_linear)
