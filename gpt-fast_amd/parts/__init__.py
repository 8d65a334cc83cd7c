"""The parts layers are made of.  Importing this package registers the built-in ones."""
from . import (attention, block, decayed_memory, differential_attention, feed_forward,  # noqa: F401
               latent_attention, matrix_memory, mixed_heads_attention, norm, position, stream_steps)
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, STREAM_STEPS, Param, Part,
                   Runtime, register_block, register_feed_forward, register_mixer, register_norm,
                   register_position, register_stream_step)
