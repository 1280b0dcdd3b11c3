"""Attention-sink mask (flaxattention/masks/attention_sink.py:6-24):
((kv_idx <= sink_size) or (q_idx - kv_idx <= window_size)) and (q_idx >= kv_idx).
Note the inclusive comparison: sink_size=4 keeps kv 0..4 visible."""
from ..core.common import INT_MIN, MaskMod
from ..core.blockmask import and_masks, or_masks
from .causal import causal_mask


def generate_attention_sink(window_size: int, sink_size: int = 4) -> MaskMod:
    sliding_window = MaskMod(lo=INT_MIN, hi=window_size, sink=-1, name="sliding_window")
    attention_sink = MaskMod(lo=INT_MIN, hi=INT_MIN, sink=sink_size, name="attention_sink")
    mask = and_masks(or_masks(attention_sink, sliding_window), causal_mask)
    mask.__name__ = f"attention_sink_{window_size}_{sink_size}"
    return mask
