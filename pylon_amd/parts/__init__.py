"""The parts layers are assembled from; importing this package registers the built-in ones."""
from . import attention, block, feed_forward, norm, position  # noqa: F401
from .base import KVRequirement, Part, StateRequirement, summed
from .registry import build_part, register_part, registered, unregister_part

__all__ = [
    "KVRequirement",
    "StateRequirement",
    "Part",
    "summed",
    "build_part",
    "register_part",
    "registered",
    "unregister_part",
]
