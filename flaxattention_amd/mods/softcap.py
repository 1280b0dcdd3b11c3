"""tanh soft-capping: cap * tanh(score / cap).  Not part of the reference; one
of the functor families the fused kernels evaluate."""
from .. import _lib
from ..core.common import ScoreMod


def generate_tanh_softcap(cap: float) -> ScoreMod:
    if not cap > 0:
        raise ValueError("cap must be positive")
    return ScoreMod(_lib.SCORE_TANH_SOFTCAP, p0=cap, p1=1.0 / cap, name=f"tanh_softcap_{cap}")
