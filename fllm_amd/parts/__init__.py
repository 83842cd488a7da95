from . import (attention, block, conv_input, embedding, experts, lightning, mlp, norm, normed_attention, pair, rope, sigmoid_attention,
               stream, talking_attention)  # noqa: F401  (register the parts)
from .base import Block, FeedForward, KVNeed, Mixer, Norm, Part, StateNeed
from .runtime import Runtime

__all__ = ["Block", "FeedForward", "KVNeed", "Mixer", "Norm", "Part", "StateNeed", "Runtime"]
