"""MI355X-native FlexAttention with the Python surface of flaxattention
(flaxattention/__init__.py:1-22)."""
from .core.attention import math_attention, flax_attention, flax_attention_pallas, kernel_family
from .core.blockmask import BlockMask, create_block_mask, create_mask, and_masks, or_masks, noop_mask
from .core.common import _mask_mod_signature, _score_mod_signature, MaskMod, ScoreMod
from .utils import visualize_attention_scores
from ._lib import FlexAttnError

__all__ = [
    "math_attention",
    "flax_attention",
    "flax_attention_pallas",
    "BlockMask",
    "create_block_mask",
    "create_mask",
    "and_masks",
    "or_masks",
    "noop_mask",
    "_mask_mod_signature",
    "_score_mod_signature",
    "visualize_attention_scores",
    "MaskMod",
    "ScoreMod",
    "FlexAttnError",
    "kernel_family",
]
