"""Parts that layers are put together from; importing this package registers the built-in kinds."""
from .base import (ARRANGEMENTS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, Block, FeedForward, Mixer, Norm, Part,
                   PositionEncoding, Rotation, Runtime, build_block, build_feed_forward, build_mixer, build_norm,
                   build_position, register_arrangement, register_feed_forward, register_mixer, register_norm,
                   register_position)
from . import attention, block, glu, norm, rope, shortconv  # noqa: F401  (registration)
from .model import DecoderModel
from .native import NativePlan
