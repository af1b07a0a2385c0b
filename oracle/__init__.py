"""CPU oracle (test infrastructure).  Python binding of oracle/libmgemv_oracle.so.

Only tests, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this package;
the shipped package mixed_gemv_amd never does.
"""
from .binding import *  # noqa: F401,F403
