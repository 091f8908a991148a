"""Grouped-query attention over the paged cache."""
from __future__ import annotations

import math

import torch

from ..config.base import ConfigError, PartSpec
from .base import (POSITION_ENCODINGS, KVCacheSpec, Mixer, PositionEncoding, WeightSpec,
                   register_mixer, to_device)


@register_mixer("gqa_attention")
class GQAttention(Mixer):
    """q, k, v projections (no bias); per-head RMS norm of q and k over the
    head size with one [d] weight each, before the rotation; the rotation; the
    keys and values of the step's tokens written to the request's pages;
    causal softmax attention with scale 1/sqrt(d) in which q head h reads kv
    head h // (nq / nkv), restricted to the last ``window`` keys if window > 0;
    output projection.

    Reference: src/core/model/qwen3/QWen3Creator.cpp:66-131 (wiring),
    src/core/model/base/ModelCreatorBase.cpp:242-283 (attention and output
    projection), src/kernel/cuda/paged_flash_attention.cu:855-1055 (kernel).
    The three projections are stacked into one [(nq + 2 nkv) d, H] matrix at
    load; the reference keeps three products (QWen3Creator.cpp:66-75).
    """

    graph_safe = True
    #: the input is used by ``ops.linear`` and by nothing else
    input_goes_to_linear = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position, qk_norm_eps: float | None = 1e-6, window: int = 0,
                 scale: float | None = None):
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        if self.num_heads % self.num_kv_heads:
            raise ConfigError(f"attention: {num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        self.qk_norm_eps = None if qk_norm_eps is None else float(qk_norm_eps)
        self.window = int(window or 0)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        if isinstance(position, PartSpec):
            position = POSITION_ENCODINGS.build(position)
        if position is not None and not isinstance(position, PositionEncoding):
            raise ConfigError("attention: 'position' must be a position encoding or its spec")
        self.position = position
        self.w_qkv = self.w_o = self.q_norm = self.k_norm = None

    def cache_spec(self):
        return KVCacheSpec(self.num_kv_heads, self.head_dim, self.window)

    def flops_per_query_key_pair(self):
        return 4 * self.num_heads * self.head_dim      # q.k and p.v, a multiply and an add each

    def weight_specs(self):
        H, nq, nkv, d = self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim
        specs = {
            "q_proj.weight": WeightSpec((nq * d, H)),
            "k_proj.weight": WeightSpec((nkv * d, H)),
            "v_proj.weight": WeightSpec((nkv * d, H)),
            "o_proj.weight": WeightSpec((H, nq * d)),
        }
        if self.qk_norm_eps is not None:
            specs["q_norm.weight"] = WeightSpec((d,), "norm")
            specs["k_norm.weight"] = WeightSpec((d,), "norm")
        return specs

    def load_weights(self, weights, dtype, device):
        qkv = torch.cat([weights["q_proj.weight"], weights["k_proj.weight"], weights["v_proj.weight"]], 0)
        self.w_qkv = to_device(qkv, dtype, device)
        self.w_o = to_device(weights["o_proj.weight"], dtype, device)
        if self.qk_norm_eps is not None:
            self.q_norm = weights["q_norm.weight"].to(torch.float32).contiguous().to(device)
            self.k_norm = weights["k_norm.weight"].to(torch.float32).contiguous().to(device)

    def forward(self, ctx, x):
        ops, kv, b = ctx.ops, ctx.kv, ctx.batch
        nq, nkv, d = self.num_heads, self.num_kv_heads, self.head_dim
        qkv = ops.linear(x, self.w_qkv)
        table = self.position.cached_table(ctx.max_positions, x.device) if self.position is not None else None
        pairing = 1 if (self.position is not None and self.position.pairing == "interleaved") else 0
        o = ops.qkv_attention(qkv, nq, nkv, d, self.q_norm, self.k_norm, self.qk_norm_eps or 0.0,
                              table, pairing, kv, b, self.window, self.scale)
        return ops.linear(o, self.w_o, out_dtype=torch.float32, partials=True)
