"""The parts layers are assembled from; importing this package registers the built-in ones."""
from . import (attention, block, delta_rule, feed_forward, latent_attention, logits, mixture, norm, parallel,  # noqa: F401
               position, retention, short_conv)
from .base import DepthMixed, KVRequirement, Normed, Part, Scaled, StateRequirement, requirement_list, summed
from .registry import build_part, register_part, registered, unregister_part

__all__ = [
    "KVRequirement",
    "StateRequirement",
    "Part",
    "Normed",
    "Scaled",
    "DepthMixed",
    "requirement_list",
    "summed",
    "build_part",
    "register_part",
    "registered",
    "unregister_part",
]
