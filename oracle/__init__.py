"""CPU oracle (test infrastructure only): ctypes access to libllmi_oracle.so.

Only tests, the smoke check and the benchmark's CPU-baseline leg may import
this package; the product path never does.
"""
from .oracle import *  # noqa: F401,F403
