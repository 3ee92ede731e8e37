"""CPU oracle for the mini-batch construction path (test infrastructure).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
import this package.  The product (apt_amd/) never does.
"""
from .oracle import *  # noqa: F401,F403
