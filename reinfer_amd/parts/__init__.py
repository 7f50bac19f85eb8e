from .base import JointNeed, KVNeed, LayerCache, PagedNeed, StateNeed, paged_need
from .registry import (lookup, register_block, register_feed_forward, register_input, register_mixer,
                       register_norm, register_position)
from . import (attention, block, decay_memory, delta_rule, feed_forward, inputs, latent_attention,  # noqa: F401  (register the parts)
               matrix_memory, moe, norm, position, side_by_side, wkv)

__all__ = ["JointNeed", "paged_need", "KVNeed", "LayerCache", "PagedNeed", "StateNeed", "lookup", "register_block", "register_feed_forward",
           "register_input", "register_mixer", "register_norm", "register_position"]
