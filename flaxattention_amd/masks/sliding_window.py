"""Sliding-window mask (flaxattention/masks/sliding_window.py:7-22):
(q_idx - kv_idx <= window_size) and (q_idx >= kv_idx)."""
from ..core.common import INT_MIN, MaskMod
from ..core.blockmask import and_masks
from .causal import causal_mask


def generate_sliding_window(window_size: int) -> MaskMod:
    sliding_window = MaskMod(lo=INT_MIN, hi=window_size, sink=-1, name="sliding_window")
    mask = and_masks(sliding_window, causal_mask)
    mask.__name__ = f"sliding_window_{window_size}"
    return mask
