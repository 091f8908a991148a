"""Qwen3 dense decoder: registration of its configuration and tensor names.

Tensor names follow the architecture's safetensors files; the reference's GGUF
names for the same tensors are ``token_embd``, ``output_norm``, ``output`` and
``blk.%d.{attn_norm, attn_q, attn_k, attn_v, attn_q_norm, attn_k_norm,
attn_output, ffn_norm, ffn_gate, ffn_up, ffn_down}``
(src/core/global/ModelGlobalVar.h:206-232).
"""
from ..config.qwen3 import ARCHITECTURE, Qwen3Config
from .decoder import TensorNames
from .registry import register_architecture

QWEN3_NAMES = TensorNames(
    embedding="model.embed_tokens",
    layer="model.layers.{i}",
    final_norm="model.norm",
    head="lm_head",
    children={
        "norm1": "input_layernorm",
        "mixer": "self_attn",
        "norm2": "post_attention_layernorm",
        "feed_forward": "mlp",
    },
)

register_architecture(ARCHITECTURE, Qwen3Config, QWEN3_NAMES)
