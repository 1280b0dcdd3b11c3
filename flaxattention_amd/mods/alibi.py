"""ALiBi (flaxattention/mods/alibi.py:5-20):
score + (q_idx - kv_idx) * exp2(-((h + 1) * 8.0 / H))."""
from .. import _lib
from ..core.common import ScoreMod


def generate_alibi_bias(H: int, sign: float = 1.0) -> ScoreMod:
    """``sign=-1`` gives slope * (kv_idx - q_idx), the spelling some
    benchmark configurations use."""
    return ScoreMod(_lib.SCORE_ALIBI, p0=sign, i0=H, name="alibi_mod")
