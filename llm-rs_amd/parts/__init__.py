from .base import (BLOCKS, FAMILIES, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, Block, FeedForward, Mixer, Norm, Part,
                   PositionEncoding, TensorSpec, build_block, build_feed_forward, build_mixer, build_norm, build_part,
                   build_position, place, register_block, register_feed_forward, register_mixer, register_norm,
                   register_part_family, register_position)
from . import attention, block, mlp, norm, rope  # noqa: F401  (register the built-in kinds)
from .attention import Attention
from .block import PreNormBlock
from .mlp import SwiGLU
from .norm import RMSNorm
from .rope import RotaryEncoding, rope_inv_freq
