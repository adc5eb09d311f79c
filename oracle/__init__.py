"""CPU oracle for the primitiv matmul path: test infrastructure only.

Only tests, the smoke check and the benchmark's CPU-baseline leg may import
this package.  The product (``primitiv_amd``) never does.
"""
from .oracle import *  # noqa: F401,F403
