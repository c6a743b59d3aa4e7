"""The parts layers are made of.  Importing this package registers the built-in ones."""
from . import attention, block, feed_forward, norm, position  # noqa: F401
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, Param, Part, Runtime,
                   register_block, register_feed_forward, register_mixer, register_norm,
                   register_position)
