from . import (attention, block, experts, feed_forward, gate, latent_attention, linear_attention, norm,  # noqa: F401  (registers the parts)
               parallel, position, readout, reentry, rotary_attention, state_space)
from .base import (Block, Delta, Embedding, FeedForward, Memory, Mixer, Norm, Part, Readout,
                   ResidualStream, Transform)
from .registry import lookup, register, unregister

__all__ = ["Block", "Delta", "Embedding", "FeedForward", "Memory", "Mixer", "Norm", "Part",
           "Readout", "ResidualStream", "Transform", "lookup", "register", "unregister"]
