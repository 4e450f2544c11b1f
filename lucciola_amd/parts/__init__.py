"""Parts of a layer: importing this package registers the built-in kinds."""
from . import attention, block, delta_rule, ends, feed_forward, input_shift, latent_attention, lightning, norm, position, stream_step  # noqa: F401
from .base import BuildContext, Part, ResidualStream, build_part  # noqa: F401
