"""Standard causal masking (flaxattention/masks/causal.py:4-5: q_idx >= kv_idx)."""
from ..core.common import INT_MAX, MaskMod

causal_mask = MaskMod(lo=0, hi=INT_MAX, sink=-1, name="causal_mask")


def offset_causal_mask(offset: int) -> MaskMod:
    """Causal mask for a query block that sits ``offset`` positions into the
    key sequence (decode: offset = KV_LEN - Q_LEN): q_idx + offset >= kv_idx."""
    return MaskMod(lo=0, hi=INT_MAX, sink=-1, q_offset=offset, name=f"offset_causal_{offset}")
