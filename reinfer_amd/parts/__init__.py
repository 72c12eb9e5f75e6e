from .base import KVNeed, LayerCache, PagedNeed, StateNeed
from .registry import (lookup, register_block, register_feed_forward, register_mixer, register_norm,
                       register_position)
from . import attention, block, feed_forward, norm, position  # noqa: F401  (register the parts)

__all__ = ["KVNeed", "LayerCache", "PagedNeed", "StateNeed", "lookup", "register_block", "register_feed_forward",
           "register_mixer", "register_norm", "register_position"]
