"""Dense gated feed-forward."""
from __future__ import annotations

import torch

from .base import FeedForward, WeightSpec, register_feed_forward, to_device


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    """f = (silu(z Wgate^T) * (z Wup^T)) Wdown^T, no biases.

    Reference: src/core/model/base/ModelCreatorBase.cpp:51-94 (up, gate, the
    unary op with x1 = gate, x2 = up, down), src/kernel/cuda/unary.cu:10-27.
    Gate and up are stacked into one [2I, H] matrix at load so that one product
    streams both; the activation reads the two halves of its rows.
    """

    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int):
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.w_gate_up = None
        self.w_down = None

    def weight_specs(self):
        H, I = self.hidden_size, self.intermediate_size
        return {
            "gate_proj.weight": WeightSpec((I, H)),
            "up_proj.weight": WeightSpec((I, H)),
            "down_proj.weight": WeightSpec((H, I)),
        }

    def load_weights(self, weights, dtype, device):
        gu = torch.cat([weights["gate_proj.weight"], weights["up_proj.weight"]], 0)
        self.w_gate_up = to_device(gu, dtype, device)
        self.w_down = to_device(weights["down_proj.weight"], dtype, device)

    def forward(self, ctx, x):
        gu = ctx.ops.linear(x, self.w_gate_up)
        m = ctx.ops.swiglu(gu)
        return ctx.ops.linear(m, self.w_down, out_dtype=torch.float32)
