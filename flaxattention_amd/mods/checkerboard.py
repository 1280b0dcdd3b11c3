"""Checkerboard score_mod (examples/benchmark.py:16-22 of the reference):
score * 0.5 where (k_idx - q_idx) is even, score * 2.0 where it is odd."""
from .. import _lib
from ..core.common import ScoreMod


def generate_checkerboard(mul_even: float = 0.5, mul_odd: float = 2.0, parity_of: str = "diff") -> ScoreMod:
    """parity_of="diff": parity of (kv_idx - q_idx) (the reference's example);
    parity_of="kv": parity of kv_idx alone."""
    if parity_of not in ("diff", "kv"):
        raise ValueError("parity_of must be 'diff' or 'kv'")
    return ScoreMod(_lib.SCORE_CHECKERBOARD, p0=mul_even, p1=mul_odd, i0=0 if parity_of == "diff" else 1,
                    name="checkerboard")


checkerboard = generate_checkerboard()
