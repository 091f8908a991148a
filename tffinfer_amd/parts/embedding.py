"""Token embedding and output head."""
from __future__ import annotations

import torch

from .base import Part, WeightSpec, to_device


class Embedding(Part):
    """x[t, :] = E[token[t], :], no scaling, into the float32 residual stream.
    Reference: src/kernel/cpu/embedding.cpp:34-49 (a CPU lookup there)."""

    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size = int(vocab_size)
        self.hidden_size = int(hidden_size)
        self.weight = None

    def weight_specs(self):
        return {"weight": WeightSpec((self.vocab_size, self.hidden_size), "embedding")}

    def load_weights(self, weights, dtype, device):
        self.weight = to_device(weights["weight"], dtype, device)

    def forward(self, ctx, token_ids):
        return ctx.ops.embed(self.weight, token_ids)


class OutputHead(Part):
    """logits = y . Wout^T in float32, no bias, no scale
    (src/core/model/qwen3/QWen3Creator.cpp:161-165, :324-329).  With tied
    embeddings the head has no tensor of its own and uses the embedding's."""

    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, tied_to: Embedding | None):
        self.vocab_size = int(vocab_size)
        self.hidden_size = int(hidden_size)
        self.tied_to = tied_to
        self._weight = None

    def weight_specs(self):
        if self.tied_to is not None:
            return {}
        return {"weight": WeightSpec((self.vocab_size, self.hidden_size), "matrix")}

    def load_weights(self, weights, dtype, device):
        if self.tied_to is None:
            self._weight = to_device(weights["weight"], dtype, device)

    @property
    def weight(self):
        return self.tied_to.weight if self.tied_to is not None else self._weight

    def forward(self, ctx, y):
        return ctx.ops.linear(y, self.weight, out_dtype=torch.float32)
