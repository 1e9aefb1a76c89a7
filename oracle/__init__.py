"""CPU oracle: numpy restatement of the reference's own numpy checks.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package imports this; it is
used by tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline leg
as the checker, never as the thing measured or shipped.
"""
from .ref_numpy import *  # noqa: F401,F403
