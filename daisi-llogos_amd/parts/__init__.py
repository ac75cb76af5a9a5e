"""Parts a layer is put together from; importing the package registers the built-in ones."""
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, Block, FeedForward, GroupView, KVSpec, LayerCache,
                   Mixer, Norm, NormedRows, Part, PositionEncoding, Residual, Runtime, StateSpec, StepContext, TensorSpec, make,
                   register_block, register_feed_forward, register_mixer, register_norm, register_position)
from .linear import Linear
from .norm import RMSNorm
from .rope import Rotary
from .attention import Attention
from .mlp import SwiGLU
from .block import PreNormBlock
