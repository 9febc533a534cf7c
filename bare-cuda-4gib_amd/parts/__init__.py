from .base import Part, register_part, build_part, registered_parts  # noqa: F401
from . import linear, norm, position, attention, feedforward, block, embedding, conv, latent_attention, rglru  # noqa: F401
from . import streams, linear_attention, diff_attention, sink_attention, reentry  # noqa: F401
