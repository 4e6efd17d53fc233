"""Parts of a decoder layer and their registries.  Importing the package
registers the built-in parts."""

from .base import (FeedForward, Mixer, Norm, PagedNeed, Part, PositionEncoding, Runtime,  # noqa: F401
                   StateNeed, TensorRule, lookup, register_arrangement, register_embedding,
                   register_feed_forward, register_head, register_mixer, register_norm,
                   register_position)
from . import norm, rope, feed_forward, embedding, attention, short_conv, block  # noqa: F401
