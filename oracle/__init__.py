"""CPU oracle for the log-probability / policy-loss path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package (`trl_amd/`) may import
this directory: only `tests/`, `__graft_entry__.smoke()` and the `cpu_baseline` leg
of `bench.py` do, and there only as the checker.
"""
from .trl_oracle import *  # noqa: F401,F403
