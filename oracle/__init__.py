"""CPU oracle for the quantized matmul path — test infrastructure only.

Only tests, the smoke check and the benchmark's CPU leg may import this
package; the shipped library never does.
"""
from .oracle import *  # noqa: F401,F403
