from .attention import Attention
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, Block, CacheBinding, CacheRequirement, DecoderSpec,
                   FeedForward, FixedState, LayerCall, Mixer, Norm, PagedKV, ParamSpec, Part, PositionEncoding,
                   Source, WEIGHT_TRANSFORMS, register_block, register_feed_forward, register_mixer, register_norm,
                   register_position_encoding, register_weight_transform)
from .block import PreNormBlock
from .embedding import Embedding, LMHead
from .rmsnorm import RMSNorm
from .rope import NoPosition, RotaryHalfSplit, rotary_tables
from .swiglu import SwiGLU
