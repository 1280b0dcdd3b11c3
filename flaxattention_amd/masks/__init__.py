"""Ready-made mask_mods (flaxattention/masks/__init__.py:1-4 re-exports
causal_mask and generate_sliding_window; generate_attention_sink lives in its
own module there and is exported here as well)."""
from .causal import causal_mask, offset_causal_mask
from .sliding_window import generate_sliding_window
from .attention_sink import generate_attention_sink

__all__ = ["causal_mask", "offset_causal_mask", "generate_sliding_window", "generate_attention_sink"]
