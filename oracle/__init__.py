"""CPU oracle for the sarek-hip hot path: TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
import this package.  The shipped library never does.
"""
from .native_oracle import *  # noqa: F401,F403
