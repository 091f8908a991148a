"""What every architecture's typed configuration has in common.

A configuration is read from the architecture's own ``config.json`` keys and
turned into two pieces of data that the rest of the engine works from:

* ``layer_specs()``: for every layer, which mixer, feed-forward, norm and block
  arrangement it is made of and with which sizes and constants;
* ``layer_schedule()``: the order in which layers run, a list that may name a
  layer twice or let a layer read another layer's cache.

The reference keeps one flat ``ModelConfig`` struct for all architectures
(src/core/model/BaseDefine.h:101-149) and copies it into a per-graph
``GraphContext`` (src/core/model/base/ModelCreatorBase.h:23-70).
"""
from __future__ import annotations

from dataclasses import dataclass, field


class ConfigError(ValueError):
    """A config.json that is incomplete, inconsistent or asks for something
    the engine does not do."""


@dataclass(frozen=True)
class PartSpec:
    """A registered part by name and the arguments it is built with."""
    kind: str
    args: dict = field(default_factory=dict)


@dataclass(frozen=True)
class LayerSpec:
    """One layer: its mixer, feed-forward and norm, and the block that arranges them."""
    block: PartSpec
    mixer: PartSpec
    feed_forward: PartSpec
    norm: PartSpec


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order.

    ``layer`` indexes ``layer_specs()``.  ``cache`` names the cache (or state)
    this call works on; two calls with the same ``cache`` share it, and
    ``writes_cache=False`` makes the call a reader of a cache another call
    fills.
    """
    layer: int
    cache: int
    writes_cache: bool = True


class ModelConfig:
    """Base of the typed configurations.  Subclasses are dataclasses."""

    architecture: str = ""

    # sizes the generic model skeleton needs
    hidden_size: int
    vocab_size: int
    max_position_embeddings: int
    tie_word_embeddings: bool

    @classmethod
    def from_dict(cls, d: dict) -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> dict:
        raise NotImplementedError

    def with_overrides(self, **values) -> "ModelConfig":
        """The configuration with some of its config.json keys replaced, checked again as
        a whole (a caller's option that overrides the file, like the reference's
        ``_rope_freq_base``, test/main.cu:26).  A key the architecture does not have is an
        error, not a silent no-op."""
        d = self.to_dict()
        unknown = [k for k in values if k not in d and not hasattr(self, k)]
        if unknown:
            raise ConfigError(f"{type(self).__name__} has no option {unknown}")
        d.update(values)
        return type(self).from_dict(d)

    def layer_specs(self) -> list[LayerSpec]:
        raise NotImplementedError

    def layer_schedule(self) -> list[LayerCall]:
        return [LayerCall(i, i) for i in range(len(self.layer_specs()))]

    def final_norm_spec(self) -> PartSpec:
        raise NotImplementedError


def require(d: dict, key: str, typ, where: str = "config.json"):
    if key not in d or d[key] is None:
        raise ConfigError(f"{where}: required key '{key}' is missing")
    return coerce(d[key], key, typ, where)


def optional(d: dict, key: str, typ, default, where: str = "config.json"):
    if key not in d or d[key] is None:
        return default
    return coerce(d[key], key, typ, where)


def coerce(v, key, typ, where):
    if typ is int:
        if isinstance(v, bool) or not isinstance(v, (int, float)) or int(v) != v:
            raise ConfigError(f"{where}: '{key}' must be an integer, found {v!r}")
        return int(v)
    if typ is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{where}: '{key}' must be a number, found {v!r}")
        return float(v)
    if typ is bool:
        if not isinstance(v, bool):
            raise ConfigError(f"{where}: '{key}' must be true or false, found {v!r}")
        return v
    if typ is str:
        if not isinstance(v, str):
            raise ConfigError(f"{where}: '{key}' must be a string, found {v!r}")
        return v
    return v
