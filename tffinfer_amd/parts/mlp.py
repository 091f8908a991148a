"""Dense gated feed-forward."""
from __future__ import annotations

import torch

from .base import FeedForward, WeightSpec, register_feed_forward, to_device


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    """f = (silu(z Wgate^T) * (z Wup^T)) Wdown^T, no biases.

    Reference: src/core/model/base/ModelCreatorBase.cpp:51-94 (up, gate, the
    unary op with x1 = gate, x2 = up, down), src/kernel/cuda/unary.cu:10-27.
    Gate and up are put into one matrix at load so that one product streams both.
    """

    graph_safe = True
    #: the input is used by ``ops.linear`` and by nothing else
    input_goes_to_linear = True

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
        gate, up = weights["gate_proj.weight"], weights["up_proj.weight"]
        if dtype == torch.bfloat16 and torch.device(device).type == "cuda":
            # bfloat16: gate and up rows interleaved in groups of 16 in one weight, so that one
            # product streams both and applies silu(gate) * up to its float32 accumulators
            from ..kernels import ops
            self.w_gate_up = ops.pack_gate_up(gate.to(dtype).contiguous().to(device),
                                              up.to(dtype).contiguous().to(device))
        else:
            # float32: gate and up stacked to [2I, H]; the activation is a kernel of its own
            self.w_gate_up = to_device(torch.cat([gate, up], 0), dtype, device)
        self.w_down = to_device(weights["down_proj.weight"], dtype, device)

    def forward(self, ctx, x):
        gu = ctx.ops.linear(x, self.w_gate_up)
        m = gu if getattr(self.w_gate_up, "glu_out", 0) else ctx.ops.swiglu(gu)
        return ctx.ops.linear(m, self.w_down, out_dtype=torch.float32, partials=True)
