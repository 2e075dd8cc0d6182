"""The parts layers are made of.  Importing this package registers the built-in ones."""
from . import (attention, block, decayed_memory, differential_attention, feed_forward,  # noqa: F401
               gated_delta, input_adds, latent_attention, matrix_memory, mixed_heads_attention, norm,
               normed_attention, parallel_mixer, position, routed_experts, sink_attention, stream_steps)
from .base import (BLOCKS, FEED_FORWARDS, INPUT_ADDS, MIXERS, NORMS, POSITIONS, STREAM_STEPS, Param,
                   Part, Runtime, register_block, register_feed_forward, register_input_add,
                   register_mixer, register_norm, register_position, register_stream_step)
