"""Head-independent relative-position bias: score + slope * (kv_idx - q_idx).
Not part of the reference; one of the functor families the fused kernels
evaluate."""
from .. import _lib
from ..core.common import ScoreMod


def generate_rel_bias(slope: float) -> ScoreMod:
    return ScoreMod(_lib.SCORE_REL_BIAS, p0=slope, name="rel_bias")
