"""Parts of a layer: importing this package registers the built-in kinds."""
from . import (attention, block, delta_rule, ends, feed_forward, input_shift, latent_attention, lightning,  # noqa: F401
               masked_attention, norm, parallel, position, state_space, stream_step)
from .base import BuildContext, Part, ResidualStream, build_part  # noqa: F401
