"""Parts layers are put together from; importing the package registers the
built-in ones."""
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, Block, FeedForward,
                   KVCacheSpec, Mixer, Norm, Part, PositionEncoding, StateSpec, WeightSpec,
                   register_block, register_feed_forward, register_mixer, register_norm,
                   register_position_encoding)
from . import attention, block, embedding, mlp, norm, position  # noqa: F401  (registration)
from .attention import GQAttention
from .block import PreNormBlock
from .embedding import Embedding, OutputHead
from .mlp import SwiGLU
from .norm import RMSNorm
from .position import NoPosition, RotaryEmbedding
