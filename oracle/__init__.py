"""CPU oracle for the FlexAttention hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; it is the checker used by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg.  It restates, in numpy / torch-CPU, the dense
algorithm of the reference's pure path (flaxattention/core/attention.py:14-106)
and its block-mask builder (flaxattention/core/blockmask.py:57-64, 253-455).
"""
from .flex_oracle import *  # noqa: F401,F403
