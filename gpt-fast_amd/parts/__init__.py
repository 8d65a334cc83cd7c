"""The parts layers are made of.  Importing this package registers the built-in ones."""
from . import (attention, block, differential_attention, feed_forward, matrix_memory,  # noqa: F401
               norm, position)
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, Param, Part, Runtime,
                   register_block, register_feed_forward, register_mixer, register_norm,
                   register_position)
