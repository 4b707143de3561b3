"""Parts of a decoder layer and their registries.  Importing the package
registers the built-in parts."""

from .base import (FeedForward, Mixer, Norm, PagedNeed, PagedStateNeed, Part, PositionEncoding, Runtime,  # noqa: F401
                   StateNeed, TensorRule, lookup, register_arrangement, register_embedding,
                   register_feed_forward, register_head, register_mixer, register_norm,
                   register_position)
from . import (norm, rope, feed_forward, experts, embedding, attention, latent_attention,  # noqa: F401
               short_conv, recurrent, block, stream)
