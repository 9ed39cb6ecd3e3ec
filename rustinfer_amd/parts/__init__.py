from .base import (FeedForward, Mixer, Norm, PagedKVNeed, ParamSpec, Part, PositionEncoding,
                   Runtime, StateNeed, stored_to)
from .norm import RMSNorm
from .rope import RotaryEmbedding, rotary_frequencies
from .linear import Linear
from .embed import Embedding, LMHead
from .mlp import SwiGLUMLP
from .attention import PagedAttention
from .block import Hidden, PreNormBlock
from .registry import (MIXERS, FEED_FORWARDS, NORMS, POSITION_ENCODINGS, register_mixer,
                       register_feed_forward, register_norm, register_position_encoding,
                       make_part)
