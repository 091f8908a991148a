"""Position encodings that rotate pairs of head elements."""
from __future__ import annotations

import math
import weakref

import torch

from ..config.base import ConfigError
from .base import PositionEncoding, register_position_encoding


@register_position_encoding("none")
class NoPosition(PositionEncoding):
    def __init__(self, head_dim: int = 0):
        self.rotary_dim = 0

    def table(self, max_positions, device):
        return None


# Rotation tables by (class, everything the law depends on, positions, device).  Layers with the same
# law share one tensor.  The entries are weak: a table lives as long as an encoding that asked for
# it does (``PositionEncoding.cached_table`` keeps it, and with it every captured decode graph that
# holds its address), and goes when the last such model goes.
_TABLES = weakref.WeakValueDictionary()


@register_position_encoding("rope")
class RotaryEmbedding(PositionEncoding):
    """angle(pos, i) = pos * theta^(-2i/rot), i < rot/2, as (cos, sin) pairs.

    Reference: the table of src/kernel/cuda/rope_table.cu:32-36
    (``pos * exp(-(2i/dim) * ln(base))``, float32 there); here the angles are
    formed in float64 on the host and the table is stored in float32.
    ``pairing='half'`` is the reference's rope type 1 (NeoX),
    'interleaved' its type 0 (src/core/model/BaseDefine.h:95-97,
    src/kernel/cuda/paged_flash_attention.cu:175-195, :343-355).
    """

    def __init__(self, head_dim: int, theta: float, pairing: str = "half",
                 rotary_dim: int | None = None):
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        self.rotary_dim = int(rotary_dim) if rotary_dim else self.head_dim
        if pairing not in ("half", "interleaved"):
            raise ConfigError(f"rope: unknown pairing '{pairing}'")
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ConfigError(f"rope: rotary size {self.rotary_dim} must be even and at most {self.head_dim}")
        self.pairing = pairing

    def angles(self, max_positions: int) -> torch.Tensor:
        half = self.rotary_dim // 2
        i = torch.arange(half, dtype=torch.float64)
        inv = torch.exp(-(2.0 * i / self.rotary_dim) * math.log(self.theta))
        return torch.arange(max_positions, dtype=torch.float64)[:, None] * inv[None, :]

    def table_key(self) -> tuple:
        """Everything ``angles`` depends on: by default all the instance's public attributes, so
        that a subclass whose law has a further parameter (a scaling factor, say) shares no table
        with an instance that has another value of it."""
        return tuple(sorted((k, v) for k, v in vars(self).items()
                            if not k.startswith("_") and isinstance(v, (int, float, str, bool, tuple, type(None)))))

    def table(self, max_positions, device):
        key = (type(self), self.table_key(), int(max_positions), str(torch.device(device)))
        t = _TABLES.get(key)
        if t is None:
            a = self.angles(max_positions)
            t = torch.stack([torch.cos(a), torch.sin(a)], -1).to(torch.float32).contiguous().to(device)
            _TABLES[key] = t
        return t
