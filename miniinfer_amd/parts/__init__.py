from .base import (BLOCKS, FEED_FORWARDS, FRAMES, MIXERS, NORMS, POSITIONS, BuildContext, FixedState, PagedKV, ParamSpec,
                   Part, Source, register_block, register_feed_forward, register_frame, register_mixer, register_norm,
                   register_position)
from . import norm, position, attention, mlp, block   # registers the built-in kinds
from .model import DecoderModel
from .norm import DeferredNorm, Norm
