"""Arrangements of mixer, feed-forward and norms in a layer."""
from __future__ import annotations

from .base import Block, register_block


@register_block("prenorm")
class PreNormBlock(Block):
    """r = x + mixer(norm1(x));  out = r + ffn(norm2(r)).

    Reference: src/core/model/qwen3/QWen3Creator.cpp:62-65 (norm before the
    mixer), :140 (first residual sum), :142-148 (norm, feed-forward), :150-151
    (second sum).  Each sum is folded into the norm that follows it: the block
    hands the feed-forward's output on as a pending term, which the next
    block's first norm (or the model's final norm) adds.
    """

    graph_safe = True

    def __init__(self, mixer, feed_forward, make_norm):
        self.norm1 = make_norm()
        self.mixer = mixer
        self.norm2 = make_norm()
        self.feed_forward = feed_forward

    def children(self):
        return {"norm1": self.norm1, "mixer": self.mixer, "norm2": self.norm2,
                "feed_forward": self.feed_forward}

    @staticmethod
    def _norm(norm, consumer, ctx, resid, pending):
        # a norm and a consumer that both say so may pass rows that still lack the norm's factor
        if getattr(norm, "for_linear_aware", False) and getattr(consumer, "input_goes_to_linear", False):
            return norm.forward(ctx, resid, pending, for_linear=True)
        return norm.forward(ctx, resid, pending)

    def forward(self, ctx, resid, pending):
        h = self._norm(self.norm1, self.mixer, ctx, resid, pending)
        a = self.mixer.forward(ctx, h)
        z = self._norm(self.norm2, self.feed_forward, ctx, resid, a)
        return self.feed_forward.forward(ctx, z)
