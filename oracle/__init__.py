"""CPU oracle loader.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this package.  The product package never does.  See refconv.c for which
reference code each function restates.
"""
from .cpu import *  # noqa: F401,F403
