"""Interfaces and registries of the parts layers are put together from.

A layer is a *block* that arranges a *mixer* (attention here), a
*feed-forward* and *norms*; a mixer may use a *position encoding*.  Every part
takes its sizes and constants as constructor arguments, says which weights it
needs (``weight_specs``), takes them (``load_weights``) and runs on the tokens
of one step (``forward``).  No part knows which model it is in: it sees only
its arguments, its weights and the step's context.

Parts are found by name in one registry per kind, so a configuration can pick
a different mixer or feed-forward for every layer, and a new part is added by
registering a class — no file of the package has to change.

The reference assembles layers from builder functions of its creator base
(``build_norm``, ``build_attn``, ``build_ffn``, ... in
src/core/model/base/ModelCreatorBase.h:116-327) and finds module classes by
string key in its ModuleFactory (include/ModuleFactory.h:89, :315-327).
"""
from __future__ import annotations

from dataclasses import dataclass, field

import torch

from ..config.base import ConfigError, PartSpec


@dataclass(frozen=True)
class WeightSpec:
    """Shape of a weight tensor and the law random weights follow:
    ``matrix`` N(0, 0.02), ``norm`` 1 + N(0, 0.1), ``embedding`` N(0, 0.02)."""
    shape: tuple
    init: str = "matrix"


@dataclass(frozen=True)
class KVCacheSpec:
    """Cache need of a mixer that keeps keys and values per token.
    ``window`` 0: all tokens are kept; > 0: only the last ``window``."""
    num_kv_heads: int
    head_dim: int
    window: int = 0


@dataclass(frozen=True)
class StateSpec:
    """Per-request state of fixed size a mixer carries from step to step."""
    shape: tuple
    dtype: torch.dtype = torch.float32


class Part:
    #: True if ``forward`` launches only kernels that take the step's sizes from
    #: device tables (no host loop over the step's entries), so that a decode step
    #: with this part can be captured in a HIP graph and replayed.  A captured step
    #: has padding rows (and runs twice on nothing but padding rows before it is
    #: captured): they write no key, and their state slot is a row of the state
    #: tensors that no request holds (``CacheManager.padding_slot``), so a part
    #: with state of its own may update the state of every row it is given.
    graph_safe = False

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {}

    def load_weights(self, weights: dict[str, torch.Tensor], dtype: torch.dtype,
                     device: torch.device) -> None:
        """``weights`` maps the names of ``weight_specs`` to host tensors in the
        type the file stores them in."""

    def children(self) -> dict[str, "Part"]:
        """Sub-parts by the name their weights are prefixed with."""
        return {}


class PositionEncoding(Part):
    """A position encoding that rotates pairs of a head's elements by angles
    that depend on the token's position.  The attention kernels take it as a
    table, so any such law (another base, scaled positions, another pairing,
    a rotated part of the head only) is a new subclass and no new kernel."""

    #: "half": pairs (i, i + rot/2); "interleaved": pairs (2i, 2i+1)
    pairing: str = "half"
    rotary_dim: int = 0

    def table(self, max_positions: int, device) -> torch.Tensor | None:
        """float32 [max_positions, rotary_dim / 2, 2] of (cos, sin), or None
        for an encoding that leaves q and k as they are."""
        raise NotImplementedError

    def cached_table(self, max_positions: int, device) -> torch.Tensor | None:
        """``table`` asked for once per (positions, device) and kept for as long as the
        encoding lives: the mixers call this, so that a subclass's ``table`` may build its
        tensor on the host each time it is called, and so that a captured decode graph,
        which holds the table's address, never sees it go."""
        cache = self.__dict__.setdefault("_table_cache", {})
        key = (int(max_positions), str(torch.device(device)))
        if key not in cache:
            cache[key] = self.table(max_positions, device)
        return cache[key]


class Norm(Part):
    def forward(self, ctx, resid: torch.Tensor, delta: torch.Tensor | None,
                rows: torch.Tensor | None = None) -> torch.Tensor:
        """Adds ``delta`` into the float32 residual stream ``resid`` (when
        ``rows`` is None) and returns the norm of the sum in the activation
        type; with ``rows`` returns the norm of those rows only.  ``delta`` is
        what a mixer or feed-forward returned: [T, hidden], or what
        ``ops.linear(..., partials=True)`` gave it: a stack [S, T, hidden] of
        partial sums to be added up or a product that has not run yet
        (``ops.add_rmsnorm`` takes all three; ``ops.as_tensor`` turns them into
        a tensor for a norm of another kind).  A norm whose class says
        ``for_linear_aware = True`` also takes ``for_linear``: the caller
        promises that the result goes to ``ops.linear`` only, so it may be rows
        that still lack the norm's per-row factor (``ops.ScaledRows``)."""
        raise NotImplementedError


class Mixer(Part):
    """Mixes information between the tokens of a request."""

    def cache_spec(self) -> KVCacheSpec | None:
        return None

    def state_spec(self) -> StateSpec | None:
        return None

    def flops_per_query_key_pair(self) -> int:
        """Flops the mixer spends on one (query token, key it reads) pair beyond its matrix
        products with weights (attention: scores and weighted values over all heads); for the
        measurements' flop counts.  0 for a mixer without such pairs."""
        return 0

    def forward(self, ctx, x: torch.Tensor) -> torch.Tensor:
        """x [T, hidden] in the activation type -> float32 [T, hidden] to be
        added to the residual stream, or what ``ops.linear(..., partials=True)``
        returns in its place for the norm that follows (``ops.as_tensor`` makes
        a tensor of it).  A mixer whose class says ``input_goes_to_linear =
        True`` hands ``x`` to ``ops.linear`` and to nothing else; it may then
        get rows that still lack their norm's factor."""
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, ctx, x: torch.Tensor) -> torch.Tensor:
        """x [T, hidden] in the activation type -> float32 [T, hidden] (or what
        ``ops.linear(..., partials=True)`` returns, as for a mixer;
        ``input_goes_to_linear`` as there)."""
        raise NotImplementedError


class Block(Part):
    """Arranges a mixer, a feed-forward and norms around the residual stream."""

    def __init__(self, mixer: Mixer, feed_forward: FeedForward, make_norm):
        raise NotImplementedError

    def forward(self, ctx, resid: torch.Tensor, pending: torch.Tensor | None) -> torch.Tensor | None:
        """``resid`` is the float32 residual stream, ``pending`` a float32 term
        the previous block has not yet added to it.  Returns the term this
        block leaves pending."""
        raise NotImplementedError


@dataclass
class Registry:
    kind: str
    classes: dict = field(default_factory=dict)

    def register(self, name: str):
        def deco(cls):
            self.classes[name] = cls
            return cls
        return deco

    def build(self, spec: PartSpec, **extra):
        try:
            cls = self.classes[spec.kind]
        except KeyError:
            raise ConfigError(
                f"unknown {self.kind} '{spec.kind}'; registered: {sorted(self.classes)}") from None
        return cls(**spec.args, **extra)


MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
NORMS = Registry("norm")
POSITION_ENCODINGS = Registry("position encoding")
BLOCKS = Registry("block")

register_mixer = MIXERS.register
register_feed_forward = FEED_FORWARDS.register
register_norm = NORMS.register
register_position_encoding = POSITION_ENCODINGS.register
register_block = BLOCKS.register


def to_device(t: torch.Tensor, dtype: torch.dtype, device):
    """A matrix to the device in ``dtype`` (float32 -> bfloat16 rounds to
    nearest even).  A bfloat16 matrix on a GPU is put into the fragment order
    the matrix-core products read (``ops.PackedWeight``); float32 stays
    row-major."""
    out = t.to(dtype).contiguous().to(device)
    if dtype == torch.bfloat16 and out.is_cuda and out.dim() == 2:
        from ..kernels import ops
        return ops.pack_weight(out)
    return out
