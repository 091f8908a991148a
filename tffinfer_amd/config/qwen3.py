"""Typed configuration of the Qwen3 dense decoder, read from its config.json.

The reference takes the same numbers from GGUF metadata
(src/core/model/gguf/GGUFLoader.cpp:244-283: embedding_length, block_count,
attention.head_count, attention.head_count_kv, attention.key_length,
feed_forward_length, attention.layer_norm_rms_epsilon) and leaves a missing key
at zero without complaint (src/core/global/ModelGlobalVar.h:1895-1897); here a
missing key without a default is an error.  The rotation base is not read from
the file there but set by the caller (test/main.cu:26); here it is
``rope_theta``.
"""
from __future__ import annotations

from dataclasses import asdict, dataclass, field

from .base import ConfigError, LayerSpec, ModelConfig, PartSpec, optional, require

ARCHITECTURE = "Qwen3ForCausalLM"


@dataclass
class Qwen3Config(ModelConfig):
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    max_position_embeddings: int
    rms_norm_eps: float = 1e-6
    rope_theta: float = 10000.0
    tie_word_embeddings: bool = False
    attention_bias: bool = False
    hidden_act: str = "silu"
    use_sliding_window: bool = False
    sliding_window: int | None = None
    max_window_layers: int | None = None
    layer_types: list[str] | None = None
    eos_token_id: int | None = None
    torch_dtype: str | None = None
    extra: dict = field(default_factory=dict, repr=False)

    architecture = ARCHITECTURE
    #: which config.json key an option of the caller overrides (the reference's _rope_freq_base)
    caller_options = {"rope_freq_base": "rope_theta"}

    @classmethod
    def from_dict(cls, d: dict) -> "Qwen3Config":
        archs = d.get("architectures")
        if not isinstance(archs, list) or not archs or archs[0] != ARCHITECTURE:
            raise ConfigError(f"config.json: 'architectures' must start with '{ARCHITECTURE}', found {archs!r}")
        H = require(d, "hidden_size", int)
        nq = require(d, "num_attention_heads", int)
        if nq <= 0:
            raise ConfigError(f"config.json: 'num_attention_heads' must be positive, found {nq}")
        eos = d.get("eos_token_id")
        if isinstance(eos, list):
            eos = eos[0] if eos else None
        known = {f for f in cls.__dataclass_fields__} | {"architectures"}
        cfg = cls(
            hidden_size=H,
            num_hidden_layers=require(d, "num_hidden_layers", int),
            num_attention_heads=nq,
            num_key_value_heads=optional(d, "num_key_value_heads", int, nq),
            head_dim=optional(d, "head_dim", int, H // nq),
            intermediate_size=require(d, "intermediate_size", int),
            vocab_size=require(d, "vocab_size", int),
            max_position_embeddings=require(d, "max_position_embeddings", int),
            rms_norm_eps=optional(d, "rms_norm_eps", float, 1e-6),
            rope_theta=optional(d, "rope_theta", float, 10000.0),
            tie_word_embeddings=optional(d, "tie_word_embeddings", bool, False),
            attention_bias=optional(d, "attention_bias", bool, False),
            hidden_act=optional(d, "hidden_act", str, "silu"),
            use_sliding_window=optional(d, "use_sliding_window", bool, False),
            sliding_window=optional(d, "sliding_window", int, None),
            max_window_layers=optional(d, "max_window_layers", int, None),
            layer_types=d.get("layer_types"),
            eos_token_id=eos if isinstance(eos, int) else None,
            torch_dtype=d.get("torch_dtype") if isinstance(d.get("torch_dtype"), str) else None,
            extra={k: v for k, v in d.items() if k not in known},
        )
        if d.get("rope_scaling") not in (None, {}):
            raise ConfigError("config.json: 'rope_scaling' is not supported (must be null)")
        cfg.validate()
        return cfg

    def validate(self) -> None:
        pos = ("hidden_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads",
               "head_dim", "intermediate_size", "vocab_size", "max_position_embeddings")
        for k in pos:
            if getattr(self, k) <= 0:
                raise ConfigError(f"config.json: '{k}' must be positive, found {getattr(self, k)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"config.json: num_attention_heads={self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads={self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"config.json: head_dim={self.head_dim} must be even for the rotation")
        if not (self.rms_norm_eps > 0):
            raise ConfigError(f"config.json: rms_norm_eps={self.rms_norm_eps} must be positive")
        if not (self.rope_theta > 0):
            raise ConfigError(f"config.json: rope_theta={self.rope_theta} must be positive")
        if self.attention_bias:
            raise ConfigError("config.json: attention_bias=true is not supported (projections have no bias)")
        if self.hidden_act != "silu":
            raise ConfigError(f"config.json: hidden_act='{self.hidden_act}' is not supported (only 'silu')")
        if self.use_sliding_window:
            if not self.sliding_window or self.sliding_window <= 0:
                raise ConfigError("config.json: use_sliding_window=true needs a positive 'sliding_window'")
        if self.layer_types is not None:
            if (not isinstance(self.layer_types, list)
                    or len(self.layer_types) != self.num_hidden_layers):
                raise ConfigError(
                    f"config.json: 'layer_types' must list {self.num_hidden_layers} layers")
            for t in self.layer_types:
                if t not in ("full_attention", "sliding_attention"):
                    raise ConfigError(f"config.json: unknown layer type '{t}'")
            if "sliding_attention" in self.layer_types and not (self.use_sliding_window and self.sliding_window):
                raise ConfigError(
                    "config.json: 'layer_types' names sliding_attention but no window is switched on")

    def to_dict(self) -> dict:
        d = asdict(self)
        extra = d.pop("extra")
        d = {k: v for k, v in d.items() if v is not None}
        d["architectures"] = [ARCHITECTURE]
        d["model_type"] = "qwen3"
        for k, v in extra.items():
            d.setdefault(k, v)
        return d

    # ---- what the layers are made of -------------------------------------
    def layer_windows(self) -> list[int]:
        """Window of each layer; 0 means every earlier key is visible.  Layers
        from ``max_window_layers`` on slide when the window is switched on,
        unless ``layer_types`` says otherwise layer by layer."""
        L = self.num_hidden_layers
        if not (self.use_sliding_window and self.sliding_window):
            return [0] * L
        types = self.layer_types
        if types is None:
            mwl = L if self.max_window_layers is None else self.max_window_layers
            types = ["sliding_attention" if i >= mwl else "full_attention" for i in range(L)]
        return [self.sliding_window if t == "sliding_attention" else 0 for t in types]

    def layer_specs(self) -> list[LayerSpec]:
        norm = PartSpec("rmsnorm", {"size": self.hidden_size, "eps": self.rms_norm_eps})
        ffn = PartSpec("swiglu", {"hidden_size": self.hidden_size,
                                  "intermediate_size": self.intermediate_size})
        specs = []
        for w in self.layer_windows():
            mixer = PartSpec("gqa_attention", {
                "hidden_size": self.hidden_size,
                "num_heads": self.num_attention_heads,
                "num_kv_heads": self.num_key_value_heads,
                "head_dim": self.head_dim,
                "qk_norm_eps": self.rms_norm_eps,
                "window": w,
                "position": PartSpec("rope", {"head_dim": self.head_dim, "theta": self.rope_theta,
                                              "pairing": "half"}),
            })
            specs.append(LayerSpec(PartSpec("prenorm", {}), mixer, ffn, norm))
        return specs

    def final_norm_spec(self) -> PartSpec:
        return PartSpec("rmsnorm", {"size": self.hidden_size, "eps": self.rms_norm_eps})
