"""Ready-made score_mods (flaxattention/mods/__init__.py:1-3 exports
generate_alibi_bias; the others are the functor families the kernels fuse)."""
from .alibi import generate_alibi_bias
from .checkerboard import checkerboard, generate_checkerboard
from .softcap import generate_tanh_softcap
from .rel_bias import generate_rel_bias

__all__ = ["generate_alibi_bias", "checkerboard", "generate_checkerboard", "generate_tanh_softcap",
           "generate_rel_bias"]
